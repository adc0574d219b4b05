"""DAG training operators of DA-Transformer on MI355X: same Python surface as
fs_plugins/custom_ops/dag_loss.py, backed by the gfx950 kernels in libdagx.so.

    dag_loss(match_all[B,T,L], links[B,L,translen], output_length[B], target_length[B]) -> [B]
    dag_best_alignment(same arguments) -> [B,L] int64
    dag_logsoftmax_gather_inplace(word_ins_out[B,L,V], select_idx[B,L,S]) -> (word_ins_out, [B,L,S] fp32)

`links` is the shifted layout (links[b,i,d] = log P(i -> i+d+1)).  Inputs may be float32,
float16 or bfloat16; all accumulation is float32 and `dag_loss` returns float32.  (float64 tensors
run through float64 kernels of their own, see float64_ops.)  Samples whose
lengths admit no path give loss -inf, zero gradients and an all -1 alignment row instead of a
device-side assert.  There is no PyTorch fallback inside these functions: without the built
library, or on a CPU tensor, they raise.
"""
import torch
from torch.autograd import Function

from .. import _native as nat
from .float64_ops import DagLossFunc64, DagLogsoftmaxGatherFunc64, best_alignment_f64

__all__ = ["dag_loss", "dag_best_alignment", "dag_logsoftmax_gather_inplace",
           "DagLossFunc", "DagBestAlignmentFunc", "DagLogsoftmaxGatherFunc", "get_dag_kernel"]


def get_dag_kernel():
    """Handle of the native library (fs_plugins/custom_ops/dag_loss.py:36-63 compiles its
    extension here; this one is built ahead of time).  Raises RuntimeError without a GPU."""
    if not torch.cuda.is_available():
        raise RuntimeError("You need GPU to use the custom DAG operations")
    return nat.lib()


_clean_workspaces = {}


def _clean_workspace(dev, nbytes):
    """Zero-filled scratch for dagx_loss_fwd.  The library needs it zero on entry and leaves it zero,
    so one buffer per (device, stream) is allocated once and handed to every call on that stream."""
    key = (dev.index, torch.cuda.current_stream(dev).cuda_stream)
    ws = _clean_workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 8), dtype=torch.uint8, device=dev)
        _clean_workspaces[key] = ws
    return ws


def _forget_workspace(dev):
    """After a failed call the buffer may hold words of an unfinished launch: the next call allocates a new one."""
    _clean_workspaces.pop((dev.index, torch.cuda.current_stream(dev).cuda_stream), None)


def _check_dag_inputs(match_all, links, output_length, target_length, who):
    if not (match_all.is_cuda and links.is_cuda and output_length.is_cuda and target_length.is_cuda):
        raise RuntimeError(f"{who}: all inputs must be GPU tensors")
    if match_all.dim() != 3 or links.dim() != 3 or output_length.dim() != 1 or target_length.dim() != 1:
        raise RuntimeError(f"{who}: match_all and links must be 3-d, the lengths 1-d")
    bsz, tarlen, prelen = match_all.shape
    if links.shape[0] != bsz or output_length.shape[0] != bsz or target_length.shape[0] != bsz:
        raise RuntimeError(f"{who}: batch size not match")
    if links.shape[1] != prelen:
        raise RuntimeError(f"{who}: links.shape[1] must equal match_all.shape[2] (graph size)")
    if output_length.dtype != torch.int64 or target_length.dtype != torch.int64:
        raise RuntimeError(f"{who}: output_length and target_length should be int64")
    if len({match_all.device, links.device, output_length.device, target_length.device}) != 1:
        raise RuntimeError(f"{who}: inputs live on different devices")
    if match_all.dtype != torch.float64 or links.dtype != torch.float64:   # (float64: kernels of their own, both tensors)
        nat.dtype_code(match_all), nat.dtype_code(links)


class DagLossFunc(Function):
    # Launch-shape selectors of the reference (fs_plugins/custom_ops/dag_loss.py:66-68); kept so
    # code that sets them keeps working, ignored by these kernels.
    config = 1
    config1 = 2
    config2 = 2
    # [B] int32 device tensor of the latest forward: whose result stands for each sample -- 0 the float32 tile
    # sweeps', 2 the float64 tile sweeps', 1 the log-domain kernel's (a diagnostic; reading it synchronises)
    last_sample_flags = None

    @staticmethod
    def forward(ctx, match_all, links, output_length, target_length):
        get_dag_kernel()
        _check_dag_inputs(match_all, links, output_length, target_length, "dag_loss")
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        links = links.contiguous()
        output_length = output_length.contiguous()
        target_length = target_length.contiguous()
        bsz, tarlen, prelen = match_all.shape
        translen = links.shape[2]
        dev = match_all.device
        nblk = (prelen + 63) // 64
        with torch.cuda.device(dev):
            # sweep results: fp32 residuals + fp64 block offsets (see include/dagx.h)
            hats = torch.empty(2, bsz, tarlen, prelen, dtype=torch.float32, device=dev)
            offs = torch.empty(2, bsz, tarlen, nblk, dtype=torch.float64, device=dev)
            logz = torch.empty(2, bsz, dtype=torch.float64, device=dev)
            # a tensor of its own, not a view of anything made here: the criterion overwrites entries of
            # the returned loss in place (fs_plugins/criterions/nat_dag_loss.py:190-191)
            loss = torch.empty(bsz, dtype=torch.float32, device=dev)
            flags = torch.empty(bsz, dtype=torch.int32, device=dev)
            nbytes = nat.workspace_bytes(nat.OP_LOSS_FWD, bsz, tarlen, prelen, translen)
            ws = _clean_workspace(dev, nbytes)
            try:
                nat.check(nat.lib().dagx_loss_fwd(
                    nat.ptr(match_all), nat.dtype_code(match_all), nat.strides3(match_all),
                    nat.ptr(links), nat.dtype_code(links), nat.ptr(output_length), nat.ptr(target_length),
                    bsz, tarlen, prelen, translen, nat.ptr(hats[0]), nat.ptr(hats[1]), nat.ptr(offs[0]), nat.ptr(offs[1]),
                    nat.ptr(logz), nat.ptr(loss), nat.ptr(flags), int(need_grad), nat.ptr(ws), nbytes, nat.stream_of(match_all)))
            except RuntimeError:
                _forget_workspace(dev)
                raise
        DagLossFunc.last_sample_flags = flags
        ctx.save_for_backward(hats, offs, logz, flags, match_all, links, output_length, target_length)
        # with gradients this is the beta read-out (the partition function the backward uses), else alpha's
        return loss

    @staticmethod
    def backward(ctx, grad_output):
        hats, offs, logz, flags, match_all, links, output_length, target_length = ctx.saved_tensors
        want_match, want_links = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        if not (want_match or want_links):
            return None, None, None, None
        bsz, tarlen, prelen = match_all.shape
        translen = links.shape[2]
        grad_output = grad_output.to(torch.float32)
        with torch.cuda.device(match_all.device):
            grad_match = torch.empty(bsz, tarlen, prelen, dtype=match_all.dtype, device=match_all.device) \
                if want_match else None
            grad_links = torch.empty_like(links) if want_links else None
            nat.check(nat.lib().dagx_loss_bwd(
                nat.ptr(grad_output), grad_output.stride(0), nat.ptr(hats[0]), nat.ptr(hats[1]),
                nat.ptr(offs[0]), nat.ptr(offs[1]), nat.ptr(logz), nat.ptr(flags),
                nat.ptr(match_all), nat.dtype_code(match_all), nat.strides3(match_all),
                nat.ptr(links), nat.dtype_code(links), nat.ptr(output_length), nat.ptr(target_length),
                bsz, tarlen, prelen, translen, nat.ptr(grad_match), nat.ptr(grad_links),
                None, 0, nat.stream_of(match_all)))
        return grad_match, grad_links, None, None


def _has_double(*tensors):
    return any(t.dtype == torch.float64 for t in tensors)


def dag_loss(match_all, links, output_length, target_length):
    """log P(target | graph) per sample, [batch] (fs_plugins/custom_ops/dag_loss.py:71-111).  float64 inputs,
    which the reference's kernels also take (dag_loss.cu:160), run through float64 kernels of their own (if only
    one of the two tensors is float64 the other is cast up): float64 arithmetic, float64 loss and gradients."""
    if _has_double(match_all, links):
        get_dag_kernel()
        match_all, links = match_all.double(), links.double()
        _check_dag_inputs(match_all, links, output_length, target_length, "dag_loss")
        return DagLossFunc64.apply(match_all, links, output_length, target_length)
    return DagLossFunc.apply(match_all, links, output_length, target_length)


class DagBestAlignmentFunc(Function):
    config = 1  # inert, see DagLossFunc

    @staticmethod
    def forward(ctx, match_all, links, output_length, target_length):
        get_dag_kernel()
        _check_dag_inputs(match_all, links, output_length, target_length, "dag_best_alignment")
        links = links.contiguous()
        output_length = output_length.contiguous()
        target_length = target_length.contiguous()
        bsz, tarlen, prelen = match_all.shape
        translen = links.shape[2]
        with torch.cuda.device(match_all.device):
            path = torch.empty(bsz, prelen, dtype=torch.int64, device=match_all.device)
            nbytes = nat.workspace_bytes(nat.OP_BEST_ALIGNMENT, bsz, tarlen, prelen, translen)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=match_all.device) if nbytes else None
            nat.check(nat.lib().dagx_best_alignment(
                nat.ptr(match_all), nat.dtype_code(match_all), nat.strides3(match_all),
                nat.ptr(links), nat.dtype_code(links), nat.ptr(output_length), nat.ptr(target_length),
                bsz, tarlen, prelen, translen, nat.ptr(path), nat.ptr(ws), nbytes, nat.stream_of(match_all)))
        ctx.mark_non_differentiable(path)
        return path

    @staticmethod
    def backward(ctx, grad_output):
        assert False, "no backward function for best alignment"


def dag_best_alignment(match_all, links, output_length, target_length):
    """Best alignment as [batch, prelen] int64 (fs_plugins/custom_ops/dag_loss.py:128-164).  float64 inputs
    (dag_best_alignment.cu:150) are scored and compared in float64, by a kernel of their own."""
    if _has_double(match_all, links):
        get_dag_kernel()
        match_all, links = match_all.detach().double(), links.detach().double()
        _check_dag_inputs(match_all, links, output_length, target_length, "dag_best_alignment")
        return best_alignment_f64(match_all, links, output_length, target_length)
    return DagBestAlignmentFunc.apply(match_all, links, output_length, target_length)


def _check_gather_inputs(word_ins_out, select_idx):
    if not (word_ins_out.is_cuda and select_idx.is_cuda):
        raise RuntimeError("dag_logsoftmax_gather_inplace: inputs must be GPU tensors")
    if word_ins_out.dim() != 3 or select_idx.dim() != 3:
        raise RuntimeError("dag_logsoftmax_gather_inplace: word_ins_out and select_idx must be 3-d")
    if not word_ins_out.is_contiguous():
        raise RuntimeError("dag_logsoftmax_gather_inplace: word_ins_out is not contiguous")
    if select_idx.dtype != torch.int64:
        raise RuntimeError("dag_logsoftmax_gather_inplace: select_idx should be int64")
    if select_idx.shape[0] != word_ins_out.shape[0] or select_idx.shape[1] != word_ins_out.shape[1]:
        raise RuntimeError("dag_logsoftmax_gather_inplace: batch size / prelen not match")


class DagLogsoftmaxGatherFunc(Function):

    @staticmethod
    def forward(ctx, word_ins_out, select_idx, transposed_storage=False):
        """Equivalent to word_ins_out.log_softmax(-1, dtype=float).gather(-1, select_idx).

        transposed_storage=True keeps the same [bsz, prelen, slen] result but stores it as
        [bsz, slen, prelen]: the criterion's next line, match.transpose(1, 2)
        (fs_plugins/criterions/nat_dag_loss.py:169, :251), then yields a contiguous [B, T, L]
        tensor, the layout the DAG kernels read with unit stride, and the gradient that comes back
        through that transpose is read in place.  Values are identical either way.

        As with the reference, word_ins_out must not be used afterwards when it requires grad:
        its storage is handed back as the gradient buffer in backward.  (The forward itself
        only reads it: the backward recomputes the probabilities from the saved per-row
        log-sum-exp instead of storing them in place.)"""
        get_dag_kernel()
        _check_gather_inputs(word_ins_out, select_idx)
        bsz, prelen, vocab = word_ins_out.shape
        slen = select_idx.shape[2]
        require_gradient = ctx.needs_input_grad[0]
        with torch.cuda.device(word_ins_out.device):
            if transposed_storage:
                selected = torch.empty(bsz, slen, prelen, dtype=torch.float32, device=word_ins_out.device).transpose(1, 2)
            else:
                selected = torch.empty(bsz, prelen, slen, dtype=torch.float32, device=word_ins_out.device)
            lse = torch.empty(bsz * prelen, dtype=torch.float32, device=word_ins_out.device) \
                if require_gradient else None
            nat.check(nat.lib().dagx_lsg_fwd(
                nat.ptr(word_ins_out), nat.dtype_code(word_ins_out), bsz, prelen, vocab, slen,
                nat.ptr(select_idx), nat.strides3(select_idx), nat.ptr(selected), nat.strides3(selected),
                nat.ptr(lse), nat.stream_of(word_ins_out)))
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
        if grad_output.dtype != torch.float32:
            grad_output = grad_output.float()
        with torch.cuda.device(grad_input.device):
            nat.check(nat.lib().dagx_lsg_bwd(
                nat.ptr(grad_input), nat.dtype_code(grad_input), bsz, prelen, vocab, slen,
                nat.ptr(select_idx), nat.strides3(select_idx), nat.ptr(grad_output), nat.strides3(grad_output),
                nat.ptr(lse), nat.stream_of(grad_input)))
        return grad_input, None, None


def dag_loss_float64_first(on=True):
    """Process-wide switch: make dag_loss start with the float64 tile sweeps for every sample instead of trying the
    float32 ones first.  For inputs known to be long and sharply peaked (a trained model's graphs of a thousand
    nodes), where the float32 sweeps' results rarely stand and their pass is lost time.  Same results to the same
    guarantee either way.  Returns the previous setting.  No counterpart in the reference (its kernels have one
    speed, fs_plugins/custom_ops/dag_loss.cu:94-127)."""
    get_dag_kernel()
    return bool(nat.lib().dagx_loss_float64_first(1 if on else 0))


def dag_logsoftmax_gather_inplace(word_ins_out, select_idx, transposed_storage=False):
    """word_ins_out.log_softmax(-1, dtype=float).gather(-1, select_idx), fused; returns
    (word_ins_out, selected) like fs_plugins/custom_ops/dag_loss.py:181-231.  See
    DagLogsoftmaxGatherFunc.forward for transposed_storage (an extension: same values, another
    memory layout of `selected`).  float64 logits (logsoftmax_gather.cu:46-58) run through a float64 kernel and give
    a float64 `selected` (logsoftmax_gather.cu:343-347)."""
    if word_ins_out.dtype == torch.float64:
        get_dag_kernel()
        _check_gather_inputs(word_ins_out, select_idx)
        return DagLogsoftmaxGatherFunc64.apply(word_ins_out, select_idx, transposed_storage)
    return DagLogsoftmaxGatherFunc.apply(word_ins_out, select_idx, transposed_storage)


@torch.no_grad()
def dag_logsoftmax_gather_argmax(word_ins_out, select_idx, transposed_storage=False):
    """The two passes over the logits at the top of glat_function
    (fs_plugins/criterions/nat_dag_loss.py:246-250) as one:
        pred_tokens = word_ins_out.argmax(-1)
        word_ins_out, match = dag_logsoftmax_gather_inplace(word_ins_out, select_idx)
    Returns (word_ins_out, selected, pred_tokens).  No gradient (the glancing pass runs without);
    the logits are only read.  Equal logits resolve to the lowest index, as torch.argmax."""
    get_dag_kernel()
    if not (word_ins_out.is_cuda and select_idx.is_cuda):
        raise RuntimeError("dag_logsoftmax_gather_argmax: inputs must be GPU tensors")
    if word_ins_out.dim() != 3 or select_idx.dim() != 3 or not word_ins_out.is_contiguous():
        raise RuntimeError("dag_logsoftmax_gather_argmax: word_ins_out must be a contiguous 3-d tensor and select_idx 3-d")
    if select_idx.dtype != torch.int64 or select_idx.shape[:2] != word_ins_out.shape[:2]:
        raise RuntimeError("dag_logsoftmax_gather_argmax: select_idx should be int64 [batch, prelen, slen]")
    bsz, prelen, vocab = word_ins_out.shape
    slen = select_idx.shape[2]
    dev = word_ins_out.device
    with torch.cuda.device(dev):
        if transposed_storage:
            selected = torch.empty(bsz, slen, prelen, dtype=torch.float32, device=dev).transpose(1, 2)
        else:
            selected = torch.empty(bsz, prelen, slen, dtype=torch.float32, device=dev)
        pred = torch.empty(bsz, prelen, dtype=torch.int64, device=dev)
        top = torch.empty(bsz, prelen, dtype=torch.float32, device=dev)
        nat.check(nat.lib().dagx_lsg_fwd_argmax(
            nat.ptr(word_ins_out), nat.dtype_code(word_ins_out), bsz, prelen, vocab, slen,
            nat.ptr(select_idx), nat.strides3(select_idx), nat.ptr(selected), nat.strides3(selected),
            None, nat.ptr(pred), nat.ptr(top), nat.stream_of(word_ins_out)))
    return word_ins_out, selected, pred


@torch.no_grad()
def dag_logsoftmax_max(output_logits):
    """output_logits.log_softmax(dim=-1).max(dim=-1) in one pass over the logits: what decoding
    takes from them (fs_plugins/models/glat_decomposed_with_link.py:900 with :692 / :721).
    Returns (values float32 [batch, prelen], tokens int64 [batch, prelen]); equal logits resolve to
    the lowest token id."""
    get_dag_kernel()
    if not output_logits.is_cuda or output_logits.dim() != 3 or not output_logits.is_contiguous():
        raise RuntimeError("dag_logsoftmax_max: output_logits must be a contiguous 3-d GPU tensor")
    bsz, prelen, vocab = output_logits.shape
    dev = output_logits.device
    with torch.cuda.device(dev):
        tokens = torch.empty(bsz, prelen, dtype=torch.int64, device=dev)
        values = torch.empty(bsz, prelen, dtype=torch.float32, device=dev)
        nat.check(nat.lib().dagx_lsg_fwd_argmax(
            nat.ptr(output_logits), nat.dtype_code(output_logits), bsz, prelen, vocab, 0,
            None, None, None, None, None, nat.ptr(tokens), nat.ptr(values), nat.stream_of(output_logits)))
    return values, tokens
