"""Decoding of the graph on the GPU: Viterbi (decode_strategy viterbi / jointviterbi,
fs_plugins/models/glat_decomposed_with_link.py:720-777: sweep, choice of the length, read-back and
token collapsing) and the greedy walk (decode_strategy greedy / lookahead, :691-718), each with one
host synchronisation at the end (the longest output)."""
from collections import namedtuple

import torch

from .. import _native as nat
from .dag_loss import get_dag_kernel

ViterbiResult = namedtuple("ViterbiResult", "output_tokens output_scores pred_length nodes")
LookaheadResult = namedtuple("LookaheadResult", "output_tokens output_scores nodes")


def _node_scores(name, links, output_logits_normalized, output_length):
    get_dag_kernel()
    if isinstance(output_logits_normalized, (tuple, list)):
        node_logp, node_tokens = output_logits_normalized
    else:
        node_logp, node_tokens = output_logits_normalized.max(dim=-1)
    if not (links.is_cuda and node_logp.is_cuda and output_length.is_cuda):
        raise RuntimeError(f"{name}: inputs must be GPU tensors")
    if links.dim() != 3 or node_logp.shape != links.shape[:2] or output_length.shape != links.shape[:1]:
        raise RuntimeError(f"{name}: links must be [batch, prelen, translen], the node scores [batch, prelen] "
                           "and output_length [batch]")
    if output_length.dtype != torch.int64 or node_tokens.dtype != torch.int64:
        raise RuntimeError(f"{name}: output_length and the node tokens must be int64")
    return node_logp.to(torch.float32).contiguous(), node_tokens.contiguous()


@torch.no_grad()
def dag_lookahead_decode(links, output_logits_normalized, output_length, decode_beta, greedy, pad_index):
    """inference_lookahead_simple on shifted links (decode_strategy lookahead, or greedy with
    greedy=True; no n-gram blocking): from node 0 always to the successor with the best
    transition + decode_beta * token log-probability, tokens collapsed on the way.
    Arguments as dag_viterbi_decode.  Returns LookaheadResult(output_tokens [batch, longest] on the
    CPU, output_scores (ones), nodes [batch, prelen]: the visited nodes, -1 after the last)."""
    node_logp, node_tokens = _node_scores("dag_lookahead_decode", links, output_logits_normalized, output_length)
    bsz, prelen, translen = links.shape
    links = links.contiguous()
    output_length = output_length.contiguous()
    with torch.cuda.device(links.device):
        out_tokens, nodes = torch.empty((2, bsz, prelen), dtype=torch.int64, device=links.device).unbind(0)
        out_count = torch.empty(bsz, dtype=torch.int64, device=links.device)
        nat.check(nat.lib().dagx_lookahead_decode(
            nat.ptr(links), nat.dtype_code(links), nat.ptr(node_logp), nat.ptr(node_tokens), nat.ptr(output_length),
            bsz, prelen, translen, float(decode_beta), int(bool(greedy)), int(pad_index),
            nat.ptr(out_tokens), nat.ptr(out_count), nat.ptr(nodes), nat.stream_of(links)))
    longest = int(out_count.max()) if bsz else 0
    output_tokens = out_tokens[:, :longest].cpu()
    return LookaheadResult(output_tokens, torch.full(output_tokens.size(), 1.0), nodes)


@torch.no_grad()
def dag_viterbi_decode(links, output_logits_normalized, output_length, decode_upsample_scale, decode_viterbibeta,
                       joint, pad_index):
    """inference_viterbi on shifted links.

    links [batch, prelen, translen]: the transitions as extract_links returns them for
    max_transition_length != -1 (no restore_valid_links needed), -inf beyond output_length;
    output_logits_normalized [batch, prelen, vocab] (or the pair (values, tokens) of its
    .max(dim=-1)); output_length int64 [batch]; joint = (decode_strategy == "jointviterbi").
    Returns ViterbiResult(output_tokens [batch, longest] padded with pad_index (a CPU tensor, as
    the reference returns), output_scores (ones), pred_length [batch], nodes [batch, max_length]:
    the path's nodes, -1 after the last).  Ties follow torch.max's first-index rule on the host."""
    node_logp, node_tokens = _node_scores("dag_viterbi_decode", links, output_logits_normalized, output_length)
    bsz, prelen, translen = links.shape
    max_length = int(2 * prelen / decode_upsample_scale)
    if max_length < 1:
        raise RuntimeError("dag_viterbi_decode: decode_upsample_scale leaves no decoding step")
    links = links.contiguous()
    output_length = output_length.contiguous()
    # the reference's penalty tensor, computed the same way on the host
    penalty = ((torch.arange(max_length) + 1) ** decode_viterbibeta).to(torch.float32).to(links.device)
    with torch.cuda.device(links.device):
        out_tokens, nodes = torch.empty((2, bsz, max_length), dtype=torch.int64, device=links.device).unbind(0)
        out_count, pred_length = torch.empty((2, bsz), dtype=torch.int64, device=links.device).unbind(0)
        nbytes = nat.workspace_bytes(nat.OP_VITERBI_DECODE, bsz, max_length, prelen, translen)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=links.device) if nbytes else None
        nat.check(nat.lib().dagx_viterbi_decode(
            nat.ptr(links), nat.dtype_code(links), nat.ptr(node_logp), nat.ptr(node_tokens), nat.ptr(output_length),
            bsz, prelen, translen, max_length, nat.ptr(penalty), int(bool(joint)), int(pad_index),
            nat.ptr(out_tokens), nat.ptr(out_count), nat.ptr(pred_length), nat.ptr(nodes),
            nat.ptr(ws), nbytes, nat.stream_of(links)))
    longest = int(out_count.max()) if bsz else 0
    output_tokens = out_tokens[:, :longest].cpu()
    return ViterbiResult(output_tokens, torch.full(output_tokens.size(), 1.0), pred_length, nodes)
