"""Transition log-probabilities from per-head scores: the tail of the link predictor
(fs_plugins/models/glat_decomposed_with_link.py:380-404, shifted branch) as one operator."""
import torch
from torch.autograd import Function

from .. import _native as nat
from .dag_loss import get_dag_kernel


def valid_end_from_tokens(prev_output_tokens, pad):
    """[B, L] exclusive end of the allowed targets for every node, from the decoder input: the
    number of non-pad tokens (the mask prev_output_tokens.ne(pad) of
    glat_decomposed_with_link.py:392 when the padding trails, as the task's collater makes it)."""
    nonpad = prev_output_tokens.ne(pad)
    lengths = nonpad.sum(-1)
    trailing = nonpad == (torch.arange(nonpad.shape[1], device=nonpad.device).unsqueeze(0) < lengths.unsqueeze(1))
    if not bool(trailing.all()):
        raise RuntimeError("dag_multihead_links: pad tokens inside a sequence are not supported")
    return lengths.unsqueeze(1).expand(-1, nonpad.shape[1]).contiguous()


def valid_end_from_bound(bound_end):
    """[B, L] exclusive end from net_input['bound_end'] (targets j <= bound_end[b, i],
    glat_decomposed_with_link.py:387-390)."""
    return (bound_end + 1).contiguous()


class DagMultiheadLinksFunc(Function):

    @staticmethod
    def forward(ctx, content, log_gates, valid_end, max_transition_length):
        get_dag_kernel()
        if not (content.is_cuda and log_gates.is_cuda and valid_end.is_cuda):
            raise RuntimeError("dag_multihead_links: inputs must be GPU tensors")
        if content.dim() != 4 or content.shape[1] != content.shape[2]:
            raise RuntimeError("dag_multihead_links: content must be [batch, prelen, prelen, heads]")
        if not content.is_contiguous():
            raise RuntimeError("dag_multihead_links: content is not contiguous")
        bsz, prelen, _, heads = content.shape
        if log_gates.shape != (bsz, prelen, heads):
            raise RuntimeError("dag_multihead_links: log_gates must be [batch, prelen, heads]")
        if valid_end.shape != (bsz, prelen) or valid_end.dtype != torch.int64:
            raise RuntimeError("dag_multihead_links: valid_end must be int64 [batch, prelen]")
        translen = int(max_transition_length)
        if translen == -1 or translen > prelen - 1:
            translen = prelen - 1
        if translen < 1:
            raise RuntimeError("dag_multihead_links: needs at least two nodes")
        gates = log_gates.detach().to(torch.float32).contiguous()
        vend = valid_end.contiguous()
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        with torch.cuda.device(content.device):
            links = torch.empty(bsz, prelen, translen, dtype=content.dtype, device=content.device)
            lse = torch.empty(bsz, prelen, heads, dtype=torch.float32, device=content.device) if need_grad else None
            nat.check(nat.lib().dagx_links_fwd(
                nat.ptr(content), nat.dtype_code(content), nat.ptr(gates), nat.ptr(vend),
                bsz, prelen, heads, translen, nat.ptr(links), nat.ptr(lse), nat.stream_of(content)))
        if need_grad:
            ctx.save_for_backward(content, gates, vend, links, lse)
            ctx.gate_dtype = log_gates.dtype
            ctx.has_backward = False
        return links

    @staticmethod
    def backward(ctx, grad_links):
        assert not ctx.has_backward, "Cannot backward twice in dag_multihead_links"
        ctx.has_backward = True
        content, gates, vend, links, lse = ctx.saved_tensors
        bsz, prelen, _, heads = content.shape
        translen = links.shape[2]
        grad_links = grad_links.to(content.dtype).contiguous()
        with torch.cuda.device(content.device):
            grad_gates = torch.empty(bsz, prelen, heads, dtype=torch.float32, device=content.device)
            # the scores' storage becomes their gradient (they are not needed by anything else:
            # the batched product that made them differentiates through its factors)
            nat.check(nat.lib().dagx_links_bwd(
                nat.ptr(content), nat.dtype_code(content), nat.ptr(gates), nat.ptr(vend),
                bsz, prelen, heads, translen, nat.ptr(links), nat.ptr(lse), nat.ptr(grad_links),
                nat.ptr(grad_gates), nat.stream_of(content)))
        # the scores have been overwritten behind autograd's back: tell it, so that any other node that saved
        # them for its own backward raises instead of differentiating through gradient values
        torch.autograd.graph.increment_version(content)
        return content, grad_gates.to(ctx.gate_dtype), None, None


def dag_multihead_links(content, log_gates, valid_end, max_transition_length):
    """links[b, i, d] = log P(i -> i+d+1) in the shifted layout the DAG operators read:
    log_softmax of every head's scores over the allowed targets inside the window, mixed over
    the heads with log_gates (logsumexp); -inf where no transition is allowed.

    content [batch, prelen, prelen, heads] (the scaled query-key products), log_gates
    [batch, prelen, heads], valid_end int64 [batch, prelen] (see valid_end_from_tokens /
    valid_end_from_bound).  As with dag_logsoftmax_gather_inplace, `content` must not be used
    afterwards when it requires grad: its storage is handed back as its gradient."""
    return DagMultiheadLinksFunc.apply(content, log_gates, valid_end, max_transition_length)
