"""Replay of the call sequence by which DA-Transformer's criterion uses the three DAG operators.

The criterion (fs_plugins/criterions/nat_dag_loss.py) and the model cannot be imported without fairseq, so
this module restates the two functions that touch the operators, with the operator set as a parameter:

    glat_function       fs_plugins/criterions/nat_dag_loss.py:239-321 (glance_strategy None)
    compute_dag_loss    fs_plugins/criterions/nat_dag_loss.py:155-203
    criterion_like      one training step: the glancing pass the model runs without gradients
                        (fs_plugins/models/glat_decomposed_with_link.py:457-461), then the main pass and
                        `loss.backward()` down to the logits and the links

What is kept exactly as the caller does it: the ids are `targets.unsqueeze(1).expand(-1, prelen, -1)` (stride 0
over the graph axis); `match` is the `transpose(1, 2)` view of the gather's output; the logits of the main pass
are a non-leaf tensor that the gather may consume in place; the alignment runs under `no_grad` on logits that
do not require grad and must come back unchanged; the returned loss is modified IN PLACE with `masked_fill_`;
the loss is `-(loss / target_length).mean()`.  The uniform random numbers of the glancing step are an argument,
so that two operator sets see the same ones.
"""
from dataclasses import dataclass
from typing import Callable

import torch

from oracle import cref
from oracle import torch_native as tn


@dataclass
class OpSet:
    gather: Callable          # (word_ins_out, select_idx) -> (word_ins_out, match [B,L,S])
    loss: Callable            # (match [B,T,L], links, output_length, target_length) -> [B]
    align: Callable           # same arguments -> [B,L] int64
    square_links: bool        # the torch_* functions take [B,L,L] links: the criterion converts first (:182-188, :265-271)
    device: str


def hip_ops(device="cuda:0", **gather_kw):
    import da_transformer_amd as dagx
    gather = (lambda w, idx: dagx.dag_logsoftmax_gather_inplace(w, idx, **gather_kw)) if gather_kw \
        else dagx.dag_logsoftmax_gather_inplace
    return OpSet(gather, dagx.dag_loss, dagx.dag_best_alignment, False, device)


def torch_oracle_ops():
    """The oracle's torch restatement of the torch_dag_* functions (CPU, small shapes)."""
    return OpSet(tn.torch_dag_logsoftmax_gather_inplace, tn.torch_dag_loss, tn.torch_dag_best_alignment, True, "cpu")


class _CrefLoss(torch.autograd.Function):
    """The float64 C oracle behind the torch_dag_loss signature, so that shapes whose torch form would
    keep (T-1) * B * L^2 autograd buffers still run through the same replay."""

    @staticmethod
    def forward(ctx, match_all, links_sq, output_length, target_length):
        loss, alpha, beta = cref.dag_loss(match_all.detach().double().numpy(), links_sq.detach().double().numpy(),
                                          output_length.numpy(), target_length.numpy())
        ctx.save_for_backward(match_all, links_sq, output_length, target_length)
        return torch.from_numpy(loss).to(match_all.dtype)

    @staticmethod
    def backward(ctx, g):
        match_all, links_sq, ol, tl = ctx.saved_tensors
        _, gm, gl = cref.dag_loss_grad(match_all.detach().double().numpy(), links_sq.detach().double().numpy(),
                                       ol.numpy(), tl.numpy(), g.double().numpy())
        return torch.from_numpy(gm).to(match_all.dtype), torch.from_numpy(gl).to(links_sq.dtype), None, None


def _cref_align(match_all, links_sq, output_length, target_length):
    path, _ = cref.best_alignment(match_all.float().numpy(), links_sq.float().numpy(), output_length.numpy(),
                                  target_length.numpy())
    return torch.from_numpy(path)


def c_oracle_ops():
    """float64 gather (torch log_softmax in float64) + the plain-C loss / alignment restatements."""
    def gather(w, idx):
        return w, torch.log_softmax(w.double(), -1).gather(-1, idx).float()
    return OpSet(gather, _CrefLoss.apply, _cref_align, True, "cpu")


def glat_function(ops, word_ins_out, tgt_tokens, prev_output_tokens, links, pad, context_p, rand,
                  force_emit=None, use_pretrain_loss=False):
    """nat_dag_loss.py:239-321.  Returns (glat_prev_output_tokens, info)."""
    prelen = links.shape[1]
    target_length = (~tgt_tokens.eq(pad)).sum(1)
    output_length = prev_output_tokens.ne(pad).sum(1)

    pred_tokens = word_ins_out.argmax(-1)                                   # :246, before the gather
    word_ins_out, match = ops.gather(word_ins_out, tgt_tokens.unsqueeze(1).expand(-1, prelen, -1))
    match = match.transpose(1, 2)

    if force_emit is None:
        force_emit = -torch.ones_like(prev_output_tokens, dtype=torch.long)
    if use_pretrain_loss:
        match = tn.force_alignment(match, force_emit)
        glat_prev_mask = force_emit >= 0
    else:
        glat_prev_mask = torch.zeros_like(prev_output_tokens, dtype=torch.bool)

    if ops.square_links:
        links = tn.restore_valid_links(links)
    path = ops.align(match, links, output_length, target_length)            # [B, prelen]

    predict_assigned_mask = path >= 0
    oracle = tgt_tokens.gather(-1, path.clip(min=0))
    same_num = ((pred_tokens == oracle) & predict_assigned_mask & ~glat_prev_mask).sum(1)
    keep_prob = ((target_length - glat_prev_mask.sum(dim=-1) - same_num) / target_length * context_p).unsqueeze(-1) \
        * predict_assigned_mask.float()
    keep_word_mask = (rand < keep_prob).bool() | glat_prev_mask
    glat_prev_output_tokens = prev_output_tokens.masked_fill(keep_word_mask, 0) + oracle.masked_fill(~keep_word_mask, 0)
    next_force_emit = path.masked_fill(~keep_word_mask, -1)
    info = {"force_emit": next_force_emit, "path": path, "pred_tokens": pred_tokens,
            "glat_accu": (same_num.sum() / target_length.sum()).detach(), "glat_keep": keep_prob.mean().detach()}
    return glat_prev_output_tokens, info


def compute_dag_loss(ops, outputs, output_masks, targets, target_masks, links, force_emit=None):
    """nat_dag_loss.py:155-203.  Returns (loss, invalid_nsentences, per-sample loss after the in-place fill)."""
    prelen = outputs.shape[1]
    output_length = output_masks.sum(dim=-1)
    target_length = target_masks.sum(dim=-1)

    outputs, match = ops.gather(outputs, targets.unsqueeze(1).expand(-1, prelen, -1))
    match = match.transpose(1, 2)
    if force_emit is not None:
        match = tn.force_alignment(match, force_emit)
    if ops.square_links:
        links = tn.restore_valid_links(links)
    loss_result = ops.loss(match, links, output_length, target_length)

    invalid_masks = loss_result.isinf().logical_or(loss_result.isnan())
    loss_result.masked_fill_(invalid_masks, 0)                               # in place, :191
    invalid_nsentences = invalid_masks.sum().detach()
    loss = -(loss_result / target_length).mean()
    return loss, invalid_nsentences, loss_result


def criterion_like(ops, logits, links, tgt_tokens, prev_output_tokens, pad, context_p, rand, force_emit=None,
                   use_pretrain_loss=False, glat=True):
    """One training step with `ops`.  logits [B,L,V] and links [B,L,translen] (shifted) are CPU tensors; they
    are moved to ops.device.  Returns a dict of CPU tensors."""
    dev = ops.device
    logits_leaf = logits.to(dev).clone().requires_grad_()
    links_leaf = links.to(dev).clone().requires_grad_()
    tgt, prev, rand = tgt_tokens.to(dev), prev_output_tokens.to(dev), rand.to(dev)
    force_emit = None if force_emit is None else force_emit.to(dev)
    out = {}
    if glat:
        with torch.no_grad():                                                 # glat_decomposed_with_link.py:457-461
            first_pass = logits_leaf.detach().clone()
            before = first_pass.clone()
            prev_glat, info = glat_function(ops, first_pass, tgt, prev, links_leaf.detach(), pad, context_p, rand,
                                            force_emit, use_pretrain_loss)
            out["logits_unchanged_by_no_grad_gather"] = bool(torch.equal(first_pass, before))
        force_emit = info["force_emit"]
        out.update(path=info["path"].cpu(), glat_tokens=prev_glat.cpu(), force_emit=force_emit.cpu(),
                   glat_accu=info["glat_accu"].cpu(), glat_keep=info["glat_keep"].cpu())
    # main pass: the decoder's outputs are non-leaf tensors
    outputs = logits_leaf * 1
    links_out = links_leaf * 1
    loss, invalid, per_sample = compute_dag_loss(ops, outputs, prev.ne(pad), tgt, tgt.ne(pad), links_out, force_emit)
    loss.backward()
    out.update(loss=loss.detach().cpu(), invalid_nsentences=invalid.cpu(), per_sample=per_sample.detach().cpu(),
               grad_logits=logits_leaf.grad.cpu(), grad_links=links_leaf.grad.cpu())
    return out


def make_step_inputs(seed, B, L, T, V, out_len, tgt_len, logits_dtype=torch.float32, links_dtype=torch.float32,
                     pad=1, logit_std=1.0, translen=None):
    """Seeded synthetic inputs of one criterion step: logits, shifted links, padded target / decoder tokens, the
    glancing step's uniform numbers."""
    import workloads
    gen = torch.Generator().manual_seed(seed)
    logits = torch.empty(B, L, V, dtype=logits_dtype)
    for b in range(B):
        logits[b] = (torch.randn(L, V, generator=gen) * logit_std).to(logits_dtype)
    links = workloads.make_links_shifted(gen, out_len, L, "cpu", dtype=links_dtype, translen=translen)
    tgt = torch.randint(4, V, (B, T), generator=gen)
    tgt = tgt.masked_fill(torch.arange(T).view(1, T) >= tgt_len.view(B, 1), pad)
    prev = torch.full((B, L), 3, dtype=torch.long).masked_fill(torch.arange(L).view(1, L) >= out_len.view(B, 1), pad)
    rand = torch.rand(B, L, generator=gen)
    return dict(logits=logits, links=links, tgt_tokens=tgt, prev_output_tokens=prev, pad=pad, rand=rand)
