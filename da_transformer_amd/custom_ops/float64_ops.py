"""The three operators for float64 tensors, backed by the float64 kernels of libdagx.so (csrc/dag_f64.hip).

The reference's extension is instantiated for double next to float and half (fs_plugins/custom_ops/dag_loss.cu:160,
dag_best_alignment.cu:150, logsoftmax_gather.cu:343-347); these are that instantiation: float64 arithmetic
throughout, float64 results and gradients.  They exist for checking -- gradcheck, a float64 run beside a float32
one -- and are plain log-domain kernels, an order of magnitude slower than the float32 operators.
The public functions of custom_ops.dag_loss send float64 tensors here.
"""
import torch
from torch.autograd import Function

from .. import _native as nat


class DagLossFunc64(Function):
    """dag_loss for float64 `match_all` and `links` (fs_plugins/custom_ops/dag_loss.py:71-120)."""

    @staticmethod
    def forward(ctx, match_all, links, output_length, target_length):
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        links = links.contiguous()
        output_length = output_length.contiguous()
        target_length = target_length.contiguous()
        bsz, tarlen, prelen = match_all.shape
        translen = links.shape[2]
        dev = match_all.device
        with torch.cuda.device(dev):
            alpha = torch.empty(bsz, tarlen, prelen, dtype=torch.float64, device=dev)
            beta = torch.empty_like(alpha) if need_grad else None
            loss = torch.empty(bsz, dtype=torch.float64, device=dev)
            nat.check(nat.lib().dagx_loss_f64_fwd(
                nat.ptr(match_all), nat.strides3(match_all), nat.ptr(links), nat.ptr(output_length), nat.ptr(target_length),
                bsz, tarlen, prelen, translen, nat.ptr(alpha), nat.ptr(beta), nat.ptr(loss), int(need_grad),
                nat.stream_of(match_all)))
        if need_grad:
            ctx.save_for_backward(alpha, beta, loss, match_all, links, output_length, target_length)
            # the criterion overwrites entries of the returned loss in place (fs_plugins/criterions/nat_dag_loss.py:190-191):
            # the backward keeps a tensor of its own
            return loss.clone()
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        alpha, beta, loss, match_all, links, output_length, target_length = ctx.saved_tensors
        want_match, want_links = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if not (want_match or want_links):
            return None, None, None, None
        bsz, tarlen, prelen = match_all.shape
        translen = links.shape[2]
        grad_output = grad_output.to(torch.float64)
        with torch.cuda.device(match_all.device):
            grad_match = torch.empty(bsz, tarlen, prelen, dtype=torch.float64, device=match_all.device) if want_match else None
            grad_links = torch.empty_like(links) if want_links else None
            nat.check(nat.lib().dagx_loss_f64_bwd(
                nat.ptr(grad_output), grad_output.stride(0), nat.ptr(alpha), nat.ptr(beta), nat.ptr(loss),
                nat.ptr(match_all), nat.strides3(match_all), nat.ptr(links), nat.ptr(output_length), nat.ptr(target_length),
                bsz, tarlen, prelen, translen, nat.ptr(grad_match), nat.ptr(grad_links), nat.stream_of(match_all)))
        return grad_match, grad_links, None, None


@torch.no_grad()
def best_alignment_f64(match_all, links, output_length, target_length):
    """dag_best_alignment for float64 tensors (fs_plugins/custom_ops/dag_loss.py:128-164): [batch, prelen] int64."""
    links = links.contiguous()
    output_length = output_length.contiguous()
    target_length = target_length.contiguous()
    bsz, tarlen, prelen = match_all.shape
    translen = links.shape[2]
    dev = match_all.device
    with torch.cuda.device(dev):
        path = torch.empty(bsz, prelen, dtype=torch.int64, device=dev)
        nbytes = nat.workspace_bytes(nat.OP_BEST_ALIGNMENT_F64, bsz, tarlen, prelen, translen)
        ws = torch.empty(max(nbytes, 8) // 8, dtype=torch.float64, device=dev)
        nat.check(nat.lib().dagx_best_alignment_f64(
            nat.ptr(match_all), nat.strides3(match_all), nat.ptr(links), nat.ptr(output_length), nat.ptr(target_length),
            bsz, tarlen, prelen, translen, nat.ptr(path), nat.ptr(ws), nbytes, nat.stream_of(match_all)))
    return path


class DagLogsoftmaxGatherFunc64(Function):
    """dag_logsoftmax_gather_inplace for float64 logits (fs_plugins/custom_ops/dag_loss.py:181-231): `selected` is
    float64; as with the other dtypes the forward only reads the logits, and the backward hands their storage back
    as the gradient."""

    @staticmethod
    def forward(ctx, word_ins_out, select_idx, transposed_storage=False):
        bsz, prelen, vocab = word_ins_out.shape
        slen = select_idx.shape[2]
        dev = word_ins_out.device
        require_gradient = ctx.needs_input_grad[0]
        with torch.cuda.device(dev):
            if transposed_storage:
                selected = torch.empty(bsz, slen, prelen, dtype=torch.float64, device=dev).transpose(1, 2)
            else:
                selected = torch.empty(bsz, prelen, slen, dtype=torch.float64, device=dev)
            lse = torch.empty(bsz * prelen, dtype=torch.float64, device=dev) if require_gradient else None
            nat.check(nat.lib().dagx_lsg_f64_fwd(
                nat.ptr(word_ins_out), bsz, prelen, vocab, slen, nat.ptr(select_idx), nat.strides3(select_idx),
                nat.ptr(selected), nat.strides3(selected), nat.ptr(lse), nat.stream_of(word_ins_out)))
        ctx.mark_dirty(word_ins_out)
        ctx.set_materialize_grads(False)
        if require_gradient:
            ctx.save_for_backward(word_ins_out, select_idx, lse)
            ctx.has_backward = False
        return word_ins_out, selected

    @staticmethod
    def backward(ctx, grad_word_ins_out, grad_output):
        if not ctx.needs_input_grad[0]:
            return None, None, None
        assert grad_word_ins_out is None, "Cannot reuse word_ins_out after logsoftmax_gather"
        if grad_output is None:
            return None, None, None
        assert not ctx.has_backward, "Cannot backward twice in logsoftmax_gather"
        ctx.has_backward = True
        grad_input, select_idx, lse = ctx.saved_tensors
        bsz, prelen, vocab = grad_input.shape
        slen = select_idx.shape[2]
        grad_output = grad_output.to(torch.float64)
        with torch.cuda.device(grad_input.device):
            nat.check(nat.lib().dagx_lsg_f64_bwd(
                nat.ptr(grad_input), bsz, prelen, vocab, slen, nat.ptr(select_idx), nat.strides3(select_idx),
                nat.ptr(grad_output), nat.strides3(grad_output), nat.ptr(lse), nat.stream_of(grad_input)))
        return grad_input, None, None
