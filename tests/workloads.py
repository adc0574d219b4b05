"""Seeded synthetic workloads for the five benchmark configurations (shared by tests and bench.py).

Generator rules: one torch.Generator per configuration seeded with 1234 + index; draws in the
fixed order lengths -> logits / match -> link logits.  Links mimic what the model's link
predictor emits (fs_plugins/models/glat_decomposed_with_link.py:387-404): log_softmax over the
valid successors i < j < L_b, -inf elsewhere, rows without a successor all -inf; they are
returned in the shifted layout [B, L, L-1] the operators take.  fp16 configurations are
generated in fp32 and rounded once, so an fp32 upcast of the same tensors is what any checker
must be fed.
"""
import torch

NEG_INF = float("-inf")


def _gen(index, device):
    g = torch.Generator(device=device)
    g.manual_seed(1234 + index)
    return g


def make_links_shifted(gen, out_len, L, device, dtype=torch.float32, translen=None, logit_scale=1.0):
    """[B,L,translen] log-probabilities built sample by sample (bounded memory)."""
    B = out_len.shape[0]
    translen = L - 1 if translen is None else min(translen, L - 1)
    i = torch.arange(L, device=device).view(L, 1)
    d = torch.arange(translen, device=device).view(1, translen)
    j = i + d + 1
    out = torch.empty(B, L, translen, dtype=dtype, device=device)
    for b in range(B):
        logits = torch.randn(L, translen, generator=gen, device=device, dtype=torch.float32) * logit_scale
        ok = j < int(out_len[b])
        logits = logits.masked_fill(~ok, NEG_INF)
        dead = ~ok.any(-1, keepdim=True)
        lp = torch.log_softmax(logits.masked_fill(dead, 0.0), -1).masked_fill(~ok, NEG_INF)
        out[b] = lp.to(dtype)
    return out


def make_match(gen, B, T, L, V, device, dtype=torch.float32, logit_std=1.0):
    """match_all [B,T,L] = log_softmax(logits [L,V])[targets], one sample at a time."""
    out = torch.empty(B, T, L, dtype=dtype, device=device)
    for b in range(B):
        logits = torch.randn(L, V, generator=gen, device=device, dtype=torch.float32) * logit_std
        targets = torch.randint(0, V, (T,), generator=gen, device=device)
        lp = torch.log_softmax(logits, -1).gather(-1, targets.view(1, T).expand(L, T))
        out[b] = lp.t().to(dtype)
    return out


def dag_config(index, device="cpu", dtype=None, rect=False, B=None, translen=None):
    """Inputs of the DAG loss / alignment configurations 0, 1, 3 and the DP part of 4.
    Returns dict(match, links (shifted), out_len, tgt_len, grad_out, V)."""
    gen = _gen(index, device)
    if index == 0:
        B0, L, T, V, dt = 4, 64, 16, 1000, torch.float32
        B = B or B0
        out_len = torch.full((B,), L, dtype=torch.long)
        tgt_len = torch.full((B,), T, dtype=torch.long)
    elif index in (1, 3):
        B0, L, T, V = 64, 512, 64, 40000
        B = B or B0
        dt = torch.float16 if index == 1 else torch.float32
        src = torch.randint(16, 65, (B,), generator=gen, device=device).cpu()
        tl = torch.randint(16, 65, (B,), generator=gen, device=device).cpu()
        if rect:
            out_len = torch.full((B,), L, dtype=torch.long)
            tgt_len = torch.full((B,), T, dtype=torch.long)
        else:
            out_len = 8 * src
            tgt_len = torch.minimum(tl, out_len)
    elif index == 4:
        B0, L, T, V, dt = 16, 1024, 256, 30522, torch.float32
        B = B or B0
        src = torch.randint(128, 257, (B,), generator=gen, device=device).cpu()
        tl = torch.randint(128, 257, (B,), generator=gen, device=device).cpu()
        out_len = 4 * src
        tgt_len = torch.minimum(tl, out_len)
    else:
        raise ValueError(index)
    dt = dtype or dt
    match = make_match(gen, B, T, L, V, device, dtype=dt)
    links = make_links_shifted(gen, out_len, L, device, dtype=dt, translen=translen)
    grad_out = (-1.0 / (B * tgt_len.double())).float()     # gradient of -mean(loss_b / T_b)
    return dict(match=match, links=links, out_len=out_len.to(device), tgt_len=tgt_len.to(device),
                grad_out=grad_out.to(device), V=V, B=B, L=L, T=T)


def gather_config(index=2, device="cpu", B=None, L=None, V=None, S=None, dtype=None):
    """Inputs of the log-softmax + gather configuration (2) or the gather part of 4."""
    gen = _gen(index, device)
    if index == 2:
        B0, L0, V0, S0, dt, std = 64, 512, 40000, 64, torch.float16, 2.0
    elif index == 4:
        B0, L0, V0, S0, dt, std = 16, 1024, 30522, 256, torch.float16, 1.0
    else:
        raise ValueError(index)
    B, L, V, S, dt = B or B0, L or L0, V or V0, S or S0, dtype or dt
    logits = torch.empty(B, L, V, dtype=dt, device=device)
    for b in range(B):
        logits[b] = (torch.randn(L, V, generator=gen, device=device, dtype=torch.float32) * std).to(dt)
    targets = torch.randint(0, V, (B, S), generator=gen, device=device)
    select_idx = targets.unsqueeze(1).expand(-1, L, -1)          # stride-0 over l, as the criterion passes it
    grad_t = torch.randn(B, S, L, generator=gen, device=device, dtype=torch.float32)
    return dict(logits=logits, targets=targets, select_idx=select_idx,
                grad_out=grad_t.transpose(1, 2), B=B, L=L, V=V, S=S)


def peaked_config(seed, B, L, T, link_scale, logit_std, V=4000, device="cpu", dtype=torch.float32, n_forced=3,
                  translen=None):
    """Inputs shaped like a trained model's: transition logits ~ N(0,1) * link_scale (one successor dominates,
    most transitions fall tens to hundreds of nats below it), token logits with standard deviation logit_std
    (wrong tokens at -30 ... -100 nats), ragged lengths, and a few nodes pinned to targets through force-emit
    rows (-inf everywhere but one node).  Returns dict(match, links (shifted), out_len, tgt_len, grad_out)."""
    gen = torch.Generator(device=device).manual_seed(seed)
    out_len = torch.randint(max(2, (3 * L) // 4), L + 1, (B,), generator=gen, device=device).cpu()
    tgt_len = torch.randint(max(2, (3 * T) // 4), T + 1, (B,), generator=gen, device=device).cpu()
    out_len[0], tgt_len[0] = L, T
    tgt_len = torch.minimum(tgt_len, out_len)
    match = make_match(gen, B, T, L, V, device, dtype=torch.float32, logit_std=logit_std)
    links = make_links_shifted(gen, out_len, L, device, dtype=dtype, translen=translen, logit_scale=link_scale)
    # pin a few nodes, spread along the diagonal so that a path exists: target t of sample b to node ~ t * L_b / T_b
    force = torch.full((B, L), -1, dtype=torch.long)
    for b in range(B):
        Lb, Tb = int(out_len[b]), int(tgt_len[b])
        for k in range(1, n_forced + 1):
            t = (k * Tb) // (n_forced + 1)
            if 0 < t < Tb - 1:
                force[b, min(Lb - 2, max(t, (t * Lb) // Tb))] = t
    hit = torch.zeros(B, T + 1, L, dtype=torch.bool).scatter_(1, force.unsqueeze(1) + 1, True)[:, 1:].to(device)
    row = hit.any(-1, keepdim=True)
    match = torch.where(row, torch.where(hit, torch.zeros_like(match), torch.full_like(match, NEG_INF)), match).to(dtype)
    grad_out = (-1.0 / (B * tgt_len.double())).float()
    return dict(match=match, links=links, out_len=out_len.to(device), tgt_len=tgt_len.to(device),
                grad_out=grad_out.to(device), B=B, L=L, T=T, force_emit=force)
