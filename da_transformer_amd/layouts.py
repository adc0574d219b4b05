"""Host-side helpers for the two link layouts and for force-emit masking.

The operators take the "shifted" layout [B, L, translen] (entry [i, d] is the transition
i -> i+d+1); the torch versions take the "square" layout [B, L, L].  These mirror what the
model and the criterion of DA-Transformer do around the operators
(fs_plugins/models/glat_decomposed_with_link.py:319-349, fs_plugins/criterions/nat_dag_loss.py:111-120).
"""
import torch

NEG_INF = float("-inf")


def _targets(prelen, translen, device):
    return torch.arange(prelen, device=device).unsqueeze(1) + torch.arange(translen, device=device).unsqueeze(0) + 1


def extract_valid_links(square, translen=None):
    """[B,L,L] -> [B,L,translen]; slots pointing past the last node are -inf."""
    bsz, prelen, _ = square.shape
    translen = prelen - 1 if translen is None else min(translen, prelen - 1)
    dst = _targets(prelen, translen, square.device)
    picked = square.gather(2, dst.clamp(max=prelen - 1).unsqueeze(0).expand(bsz, -1, -1))
    return picked.masked_fill((dst >= prelen).unsqueeze(0), NEG_INF)


def restore_valid_links(links):
    """[B,L,translen] -> [B,L,L] with -inf wherever no transition is stored."""
    bsz, prelen, translen = links.shape
    dst = _targets(prelen, translen, links.device).clamp(max=prelen)
    wide = links.new_full((bsz, prelen, prelen + 1), NEG_INF)
    wide.scatter_(2, dst.unsqueeze(0).expand(bsz, -1, -1), links)
    return wide[:, :, :prelen]


def force_alignment(match, force_emit):
    """Rows of `match` [B,T,L] whose target is pinned by force_emit[b,j] = t >= 0 become 0 at
    node j and -inf elsewhere (and stop carrying gradient); other rows pass through."""
    bsz, tarlen, prelen = match.shape
    hit = torch.zeros(bsz, tarlen + 1, prelen, dtype=torch.bool, device=match.device)
    hit.scatter_(1, force_emit.unsqueeze(1) + 1, True)
    hit = hit[:, 1:]
    forced = hit.any(dim=-1, keepdim=True)
    pinned = torch.zeros_like(match).masked_fill_(~hit, NEG_INF).masked_fill_(~forced, 0.0)
    return match.masked_fill(forced, 0.0) + pinned
