"""Small seeded input builders shared by the CPU and GPU tests."""
import torch

from oracle import torch_native as tn

NEG_INF = float("-inf")


def random_links_square(gen, B, L, out_len, dtype=torch.float64, drop=0.0, translen=None):
    """log_softmax over valid successors j in (i, L_b) (optionally j-i <= translen), -inf elsewhere;
    rows without a successor are all -inf.  `drop` masks extra edges at random (kept rows stay
    normalised over the surviving edges)."""
    logits = torch.randn(B, L, L, generator=gen, dtype=torch.float64)
    i = torch.arange(L).view(1, L, 1)
    j = torch.arange(L).view(1, 1, L)
    ok = (j > i) & (j < out_len.view(B, 1, 1))
    if translen is not None:
        ok = ok & (j - i <= translen)
    if drop > 0:
        keep = torch.rand(B, L, L, generator=gen) >= drop
        keep = keep | (j == i + 1)  # never cut the chain 0,1,2,... so a path always exists
        ok = ok & keep
    logits = logits.masked_fill(~ok, NEG_INF)
    dead = ~ok.any(-1, keepdim=True)
    out = torch.log_softmax(logits.masked_fill(dead, 0.0), -1).masked_fill(~ok, NEG_INF)
    return out.to(dtype)


def random_problem(seed, B, L, T, dtype=torch.float64, ragged=True, drop=0.0, translen=None,
                   match_scale=1.0):
    gen = torch.Generator().manual_seed(seed)
    if ragged:
        out_len = torch.randint(max(2, L - 4), L + 1, (B,), generator=gen)
        tgt_len = torch.randint(max(2, T - 3), T + 1, (B,), generator=gen)
        tgt_len = torch.minimum(tgt_len, out_len)
    else:
        out_len = torch.full((B,), L, dtype=torch.long)
        tgt_len = torch.full((B,), T, dtype=torch.long)
    match = (torch.randn(B, T, L, generator=gen, dtype=torch.float64) * match_scale - 2.0).to(dtype)
    links = random_links_square(gen, B, L, out_len, dtype=dtype, drop=drop, translen=translen)
    return match, links, out_len, tgt_len


def path_nodes(path_row):
    """[L] tensor of t-or-(-1)  ->  list of node indices ordered by t."""
    pairs = [(int(t), j) for j, t in enumerate(path_row.tolist()) if t >= 0]
    pairs.sort()
    return [j for _, j in pairs]


def shifted(links_sq, translen=None):
    return tn.extract_valid_links(links_sq, translen)
