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


def make_links_shifted(gen, out_len, L, device, dtype=torch.float32, translen=None):
    """[B,L,translen] log-probabilities built sample by sample (bounded memory)."""
    B = out_len.shape[0]
    translen = L - 1 if translen is None else min(translen, L - 1)
    i = torch.arange(L, device=device).view(L, 1)
    d = torch.arange(translen, device=device).view(1, translen)
    j = i + d + 1
    out = torch.empty(B, L, translen, dtype=dtype, device=device)
    for b in range(B):
        logits = torch.randn(L, translen, generator=gen, device=device, dtype=torch.float32)
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
