"""The criterion's glue around the DAG operators as single launches: pinning nodes to targets
(fs_plugins/criterions/nat_dag_loss.py:111-120) and glancing after the best alignment
(fs_plugins/criterions/nat_dag_loss.py:273-311)."""
from collections import namedtuple

import torch
from torch.autograd import Function

from .. import _native as nat
from .dag_loss import get_dag_kernel


def _force_emit(match, force_emit, gradient):
    bsz, tarlen, prelen = match.shape
    out = torch.empty(bsz, tarlen, prelen, dtype=match.dtype, device=match.device)
    with torch.cuda.device(match.device):
        nat.check(nat.lib().dagx_force_emit(
            nat.ptr(match), nat.dtype_code(match), nat.strides3(match), nat.ptr(force_emit),
            bsz, tarlen, prelen, int(gradient), nat.ptr(out), nat.stream_of(match)))
    return out


class DagForceAlignmentFunc(Function):

    @staticmethod
    def forward(ctx, match, force_emit):
        get_dag_kernel()
        if not (match.is_cuda and force_emit.is_cuda):
            raise RuntimeError("dag_force_alignment: inputs must be GPU tensors")
        if match.dim() != 3 or force_emit.shape != (match.shape[0], match.shape[2]):
            raise RuntimeError("dag_force_alignment: match must be [batch, tarlen, prelen] and force_emit [batch, prelen]")
        if force_emit.dtype != torch.int64:
            raise RuntimeError("dag_force_alignment: force_emit must be int64")
        force_emit = force_emit.contiguous()
        ctx.save_for_backward(force_emit)
        return _force_emit(match, force_emit, False)

    @staticmethod
    def backward(ctx, grad):
        force_emit, = ctx.saved_tensors
        return _force_emit(grad, force_emit, True), None


def dag_force_alignment(match, force_emit):
    """NATDAGLoss._force_aligment: if force_emit[b, j] = t >= 0, row t of match[b] becomes 0 at
    node j and -inf at every other node; rows no node names pass through.  Named rows carry no
    gradient.  match [batch, tarlen, prelen] (any strides), force_emit int64 [batch, prelen]
    with values in [-1, tarlen)."""
    return DagForceAlignmentFunc.apply(match, force_emit)


GlatGlance = namedtuple("GlatGlance", "oracle same_num keep_prob keep_word_mask glat_prev_output_tokens next_force_emit")


def _check_glat(name, path, **tensors):
    get_dag_kernel()
    if path.dim() != 2 or path.dtype != torch.int64 or not path.is_cuda:
        raise RuntimeError(f"{name}: path must be an int64 GPU tensor [batch, prelen]")
    for what, (t, dtype, shape) in tensors.items():
        if t is None:
            continue
        if not t.is_cuda or t.dtype != dtype or (shape is not None and tuple(t.shape) != shape):
            raise RuntimeError(f"{name}: {what} must be a {dtype} GPU tensor of shape {shape}")


def dag_glat_oracle(path, tgt_tokens, pred_tokens, glat_prev_mask=None):
    """oracle[b, j] = tgt_tokens[b, max(path[b, j], 0)] and same_num[b] = the assigned, not
    pinned nodes whose prediction already is that token (nat_dag_loss.py:273-275)."""
    bsz, prelen = path.shape
    _check_glat("dag_glat_oracle", path,
                tgt_tokens=(tgt_tokens, torch.int64, None), pred_tokens=(pred_tokens, torch.int64, (bsz, prelen)),
                glat_prev_mask=(glat_prev_mask, torch.bool, (bsz, prelen)))
    if tgt_tokens.dim() != 2 or tgt_tokens.shape[0] != bsz:
        raise RuntimeError("dag_glat_oracle: tgt_tokens must be [batch, tarlen]")
    path, tgt_tokens, pred_tokens = path.contiguous(), tgt_tokens.contiguous(), pred_tokens.contiguous()
    mask = None if glat_prev_mask is None else glat_prev_mask.contiguous()
    with torch.cuda.device(path.device):
        oracle = torch.empty_like(path)
        same_num = torch.empty(bsz, dtype=torch.int64, device=path.device)
        nat.check(nat.lib().dagx_glat_glance(
            nat.ptr(path), nat.ptr(tgt_tokens), nat.ptr(pred_tokens), None, nat.ptr(mask), None,
            None, None, 0.0, bsz, tgt_tokens.shape[1], prelen, 1,
            nat.ptr(oracle), nat.ptr(same_num), None, None, None, None, nat.stream_of(path)))
    return oracle, same_num


def dag_glat_mix(path, oracle, prev_output_tokens, keep_prob, rand, glat_prev_mask=None):
    """keep_word_mask = rand < keep_prob | glat_prev_mask, the second pass's decoder input
    (oracle token on kept nodes) and its force_emit (path on kept nodes, else -1)
    (nat_dag_loss.py:307-311).  Returns (keep_word_mask, glat_prev_output_tokens, next_force_emit)."""
    bsz, prelen = path.shape
    shape = (bsz, prelen)
    _check_glat("dag_glat_mix", path, oracle=(oracle, torch.int64, shape),
                prev_output_tokens=(prev_output_tokens, torch.int64, shape), keep_prob=(keep_prob, torch.float32, shape),
                rand=(rand, torch.float32, shape), glat_prev_mask=(glat_prev_mask, torch.bool, shape))
    path, oracle, prev = path.contiguous(), oracle.contiguous(), prev_output_tokens.contiguous()
    keep_prob, rand = keep_prob.contiguous(), rand.contiguous()
    mask = None if glat_prev_mask is None else glat_prev_mask.contiguous()
    with torch.cuda.device(path.device):
        keep = torch.empty(shape, dtype=torch.bool, device=path.device)
        tokens = torch.empty_like(path)
        force = torch.empty_like(path)
        nat.check(nat.lib().dagx_glat_glance(
            nat.ptr(path), None, None, nat.ptr(prev), nat.ptr(mask), None,
            nat.ptr(rand), nat.ptr(keep_prob), 0.0, bsz, 1, prelen, 2,
            nat.ptr(oracle), None, None, nat.ptr(keep), nat.ptr(tokens), nat.ptr(force), nat.stream_of(path)))
    return keep, tokens, force


def dag_glat_glance(path, tgt_tokens, pred_tokens, prev_output_tokens, target_length, context_p,
                    glat_prev_mask=None, rand=None):
    """Everything glat_function does between dag_best_alignment and its return, for
    glance_strategy None (nat_dag_loss.py:273-278, 307-311), in one launch: every assigned node is
    revealed with probability (T_b - pinned - same_num) / T_b * context_p.  `rand` [batch, prelen]
    uniform float32 (drawn with torch.rand when not given, as the criterion draws it).
    Returns GlatGlance(oracle, same_num, keep_prob, keep_word_mask, glat_prev_output_tokens,
    next_force_emit)."""
    bsz, prelen = path.shape
    shape = (bsz, prelen)
    if rand is None:
        rand = torch.rand(shape, device=path.device)
    _check_glat("dag_glat_glance", path,
                tgt_tokens=(tgt_tokens, torch.int64, None), pred_tokens=(pred_tokens, torch.int64, shape),
                prev_output_tokens=(prev_output_tokens, torch.int64, shape), target_length=(target_length, torch.int64, (bsz,)),
                rand=(rand, torch.float32, shape), glat_prev_mask=(glat_prev_mask, torch.bool, shape))
    if tgt_tokens.dim() != 2 or tgt_tokens.shape[0] != bsz:
        raise RuntimeError("dag_glat_glance: tgt_tokens must be [batch, tarlen]")
    path, tgt_tokens, pred_tokens = path.contiguous(), tgt_tokens.contiguous(), pred_tokens.contiguous()
    prev, target_length, rand = prev_output_tokens.contiguous(), target_length.contiguous(), rand.contiguous()
    mask = None if glat_prev_mask is None else glat_prev_mask.contiguous()
    with torch.cuda.device(path.device):
        oracle, tokens, force = torch.empty((3,) + shape, dtype=torch.int64, device=path.device).unbind(0)
        same_num = torch.empty(bsz, dtype=torch.int64, device=path.device)
        keep_prob = torch.empty(shape, dtype=torch.float32, device=path.device)
        keep = torch.empty(shape, dtype=torch.bool, device=path.device)
        nat.check(nat.lib().dagx_glat_glance(
            nat.ptr(path), nat.ptr(tgt_tokens), nat.ptr(pred_tokens), nat.ptr(prev), nat.ptr(mask), nat.ptr(target_length),
            nat.ptr(rand), None, float(context_p), bsz, tgt_tokens.shape[1], prelen, 3,
            nat.ptr(oracle), nat.ptr(same_num), nat.ptr(keep_prob), nat.ptr(keep), nat.ptr(tokens), nat.ptr(force),
            nat.stream_of(path)))
    return GlatGlance(oracle, same_num, keep_prob, keep, tokens, force)
