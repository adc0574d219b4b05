"""Pure-PyTorch versions of the three operators (square link layout), selectable by the caller
exactly like DA-Transformer's --torch-dag-loss / --torch-dag-best-alignment /
--torch-dag-logsoftmax-gather switches (fs_plugins/custom_ops/dag_loss.py:237-359).

They are public API for callers that ask for them by name.  The HIP operators in dag_loss.py
never route through this file.
"""
import torch

_NEG_INF = float("-inf")


def logsumexp_keepdim(x, dim: int):
    """logsumexp(keepdim=True) whose all -inf slices give -inf with zero gradient
    (fs_plugins/custom_ops/dag_loss.py:237-245)."""
    peak = x.max(dim=dim, keepdim=True)[0].detach()
    empty = peak == _NEG_INF
    ref = peak.masked_fill(empty, 0.0)
    acc = (x - ref).exp().sum(dim=dim, keepdim=True)
    return acc.masked_fill(empty, 1.0).log() + ref.masked_fill(empty, _NEG_INF)


def _sweep(match_all, links, output_length, target_length, reduce_fn):
    if links.dim() != 3 or links.shape[1] != links.shape[2]:
        raise AssertionError("links should be batch_size * prelen * prelen")
    bsz, tarlen, prelen = match_all.shape
    state = torch.full((bsz, prelen), _NEG_INF, dtype=match_all.dtype, device=match_all.device)
    state[:, 0] = match_all[:, 0, 0]
    history = [state]
    for step in range(1, tarlen):
        state = reduce_fn(state.unsqueeze(2) + links) + match_all[:, step]
        history.append(state)
    table = torch.stack(history, 1)
    return table[torch.arange(bsz, device=table.device), target_length - 1, output_length - 1]


def torch_dag_loss(match_all, links, output_length, target_length):
    """Log-likelihood of the target under the DAG; links [B,L,L], match_all [B,T,L]
    (fs_plugins/custom_ops/dag_loss.py:259-300)."""
    return _sweep(match_all, links, output_length, target_length,
                  lambda scores: logsumexp_keepdim(scores, 1).squeeze(1))


def _torch_max_loss(match_all, links, output_length, target_length):
    return _sweep(match_all, links, output_length, target_length,
                  lambda scores: torch.max(scores, dim=1)[0])


def torch_dag_best_alignment(match_all, links, output_length, target_length):
    """[B,L] int64 alignment (target index per node, -1 off the path); ties go to the lowest
    predecessor index (fs_plugins/custom_ops/dag_loss.py:322-353)."""
    with torch.enable_grad():
        probe = match_all.detach().requires_grad_()
        best = _torch_max_loss(probe, links.detach(), output_length, target_length)
        visits = torch.autograd.grad(best.sum(), [probe])[0]
    strength, path = visits.max(dim=1)
    return path.masked_fill_(strength < 0.5, -1)


def torch_dag_logsoftmax_gather_inplace(word_ins_out, select_idx):
    """log_softmax (fp32) + gather; leaves word_ins_out untouched
    (fs_plugins/custom_ops/dag_loss.py:355-359)."""
    picked = torch.log_softmax(word_ins_out, -1, dtype=torch.float32).gather(-1, select_idx)
    return word_ins_out, picked
