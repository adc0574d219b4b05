#!/usr/bin/env python3
"""Benchmark of the DAG training operators on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--skip-cpu] [--skip-gather] [--leg NAME]

One "step" is DAG-loss forward + backward (public Python API, autograd included) on one
synthetic batch of the headline shape B=64, L=512, T=64 (all samples full length, fp16 inputs,
fp32 accumulation), inputs resident in HBM: `value` = samples/s over the timed steps.  The same
run also times, with HIP events on the launch stream, the individual operators through the C ABI:

  roofline         the tile sweeps of the forward (the headline's dominant kernel) against the
                   vector-ALU roof, HBM bytes per launch read from the committed traffic profile
  roofline_dp      sweeps + gradient kernels against the same roof (frac: the two timed one by one;
                   frac_over_timed_steps: the same work over the timed steps of `value`)
  roofline_gather  log-softmax + gather backward (and forward) at [64,512,40000] fp16 against 8 TB/s
  dag_other_workloads   ragged lengths, the reference tuner's shape, inputs like a trained model's
  cpu_baseline     the torch-native restatement on the host cores (a bounded sample)

and the alignment, the link predictor's tail, the criterion glue, decoding, the criterion sequence of
configuration 4 and the torch-native path on the same GPU.  `--leg dag` / `--leg gather` / ... run one
part only (profiling aid; the dag leg ends with three plain device copies of known size, the
calibration dispatches for the HBM byte counters).  Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
VALU_PEAK_LANEOPS = 256 * 64 * 2.4e9   # 256 CUs x 64 fp32 lanes x 2.4 GHz (single issue)
CALIBRATION_COPY_BYTES = 1 << 30       # the --leg dag run ends with three plain device copies of this size


def profile_table_row(filename, row_prefix):
    """Cells of the first table row of profiles/<filename> whose first cell starts with row_prefix (None when the
    file or the row is missing): the HBM-traffic figures of the roofline objects are read from the committed
    rocprofv3 summaries, not typed in here."""
    path = os.path.join(ROOT, "profiles", filename)
    if not os.path.exists(path):
        return None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if line.startswith("|") and cells and cells[0].strip("`").startswith(row_prefix):
            return cells
    return None


def profile_source_revision(filename):
    """The source revision a profiles/ summary says it was taken at (its "Source revision:" line), or None."""
    path = os.path.join(ROOT, "profiles", filename)
    if not os.path.exists(path):
        return None
    for line in open(path):
        if line.startswith("Source revision:"):
            return line.split(":", 1)[1].strip()
    return None


def traffic_bytes(filename, row_prefix, fetched_col, written_col):
    """fetched + written bytes per launch from a profiles/*_hbm_traffic.md table ("2.699 GB" style cells)."""
    cells = profile_table_row(filename, row_prefix)
    if not cells:
        return None
    try:
        return (float(cells[fetched_col].split()[0]) + float(cells[written_col].split()[0])) * 1e9
    except (ValueError, IndexError):
        return None


def event_time_ms(fn, iters, warmup=5, rounds=3):
    """Average duration of fn() in ms, HIP events on torch's current stream (the launch stream):
    the median over `rounds` back-to-back rounds of `iters` calls (the first round after an idle
    spell runs at lower clocks)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(rounds):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(iters):
            fn()
        stop.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(stop) / iters)
    return sorted(times)[len(times) // 2]


def pair_updates(out_len, tgt_len, translen):
    """U = sum_b (T_b-1) * #{(i,j): i<j<L_b, j-i<=translen}."""
    total = 0
    for Lb, Tb in zip(out_len.tolist(), tgt_len.tolist()):
        w = min(translen, Lb - 1)
        pairs = w * Lb - w * (w + 1) // 2
        total += (Tb - 1) * pairs
    return total


def gather_leg(args, torch, nat, lib, stream, workloads, dev):
    """log-softmax + gather at [64,512,40000] fp16 through the C ABI; returns (roofline, details)."""
    g = workloads.gather_config(2, device=dev)
    x, idx, gsel = g["logits"], g["select_idx"], g["grad_out"]
    Bg, Lg, V, S = g["B"], g["L"], g["V"], g["S"]
    sel = torch.empty(Bg, Lg, S, device=dev); lse = torch.empty(Bg * Lg, device=dev)
    dt = nat.dtype_code(x)
    is3, ss3, gs3 = nat.strides3(idx), nat.strides3(sel), nat.strides3(gsel)

    def lsg_fwd():
        nat.check(lib.dagx_lsg_fwd(x.data_ptr(), dt, Bg, Lg, V, S, idx.data_ptr(), is3, sel.data_ptr(), ss3,
                                   lse.data_ptr(), stream))

    def lsg_bwd():   # in place; the buffer keeps holding valid numbers, timing is value independent
        nat.check(lib.dagx_lsg_bwd(x.data_ptr(), dt, Bg, Lg, V, S, idx.data_ptr(), is3, gsel.data_ptr(), gs3,
                                   lse.data_ptr(), stream))
    pred = torch.empty(Bg, Lg, dtype=torch.int64, device=dev); top = torch.empty(Bg, Lg, device=dev)

    def lsg_fwd_argmax():   # the same pass also yields word_ins_out.argmax(-1) (nat_dag_loss.py:246)
        nat.check(lib.dagx_lsg_fwd_argmax(x.data_ptr(), dt, Bg, Lg, V, S, idx.data_ptr(), is3, sel.data_ptr(), ss3,
                                          lse.data_ptr(), pred.data_ptr(), top.data_ptr(), stream))

    def lsg_max_only():     # decoding: log_softmax(-1).max(-1) (glat_decomposed_with_link.py:900, :721)
        nat.check(lib.dagx_lsg_fwd_argmax(x.data_ptr(), dt, Bg, Lg, V, 0, None, None, None, None, None,
                                          pred.data_ptr(), top.data_ptr(), stream))
    n = max(5, min(args.steps, 20))   # (the side legs are event-timed: 20 repetitions are enough)
    fwd_ms = event_time_ms(lsg_fwd, n)
    fwd_argmax_ms = event_time_ms(lsg_fwd_argmax, n)
    max_only_ms = event_time_ms(lsg_max_only, n)
    torch_argmax_ms = event_time_ms(lambda: x.argmax(-1), 3, warmup=1, rounds=1)
    torch_logsoftmax_max_ms = event_time_ms(lambda: x.log_softmax(dim=-1).max(dim=-1), 3, warmup=1, rounds=1)
    bwd_ms = event_time_ms(lsg_bwd, n)
    # plain device copy of the same buffer: the calibration kernel for the HBM byte counters
    y = torch.empty_like(x)
    copy_ms = event_time_ms(lambda: y.copy_(x), n)
    nbytes = x.numel() * x.element_size()
    small = Bg * Lg * S * 4
    fwd_gbs = (nbytes + small) / (fwd_ms * 1e-3) / 1e9
    bwd_gbs = (2 * nbytes + small) / (bwd_ms * 1e-3) / 1e9
    both_gbs = (3 * nbytes + 2 * small) / ((fwd_ms + bwd_ms) * 1e-3) / 1e9
    # HBM bytes per launch of this kernel on this workload: rocprofv3 FETCH_SIZE / WRITE_SIZE runs scaled by a
    # plain device copy of the same buffer, read from the committed summary
    same_shape = (Bg, Lg, V, S, x.element_size()) == (64, 512, 40000, 64, 2)
    traffic = traffic_bytes("lsg_fp16_64x512x40000_hbm_traffic.md", "dagx::lsg_bwd_kernel", 3, 4) if same_shape else None
    fwd_traffic = traffic_bytes("lsg_fp16_64x512x40000_hbm_traffic.md", "dagx::lsg_fwd_kernel<__half, 512, 2, false>", 3, 4) if same_shape else None
    roofline = {"kernel": "lsg_bwd_kernel<half>", "bound": "hbm", "achieved": bwd_gbs, "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": bwd_gbs / HBM_PEAK_GBS, "traffic": traffic,
                "algorithmic_bytes": 2 * nbytes + small, "kernel_ms": bwd_ms,
                "forward": {"kernel": "lsg_fwd_kernel<half>", "achieved": fwd_gbs, "frac": fwd_gbs / HBM_PEAK_GBS,
                            "traffic": fwd_traffic, "algorithmic_bytes": nbytes + small, "kernel_ms": fwd_ms}}
    gather = {"workload": "logsoftmax_gather [64,512,40000] fp16, S=64 (stride-0 ids)",
              "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "fwd_GBps": fwd_gbs, "bwd_GBps": bwd_gbs,
              "fwd_bwd_GBps": both_gbs, "fwd_frac_of_peak": fwd_gbs / HBM_PEAK_GBS,
              "fwd_bwd_frac_of_peak": both_gbs / HBM_PEAK_GBS,
              "fwd_with_argmax_ms": fwd_argmax_ms, "torch_argmax_ms_same_gpu": torch_argmax_ms,
              "logsoftmax_max_ms": max_only_ms, "torch_logsoftmax_then_max_ms_same_gpu": torch_logsoftmax_max_ms,
              "plain_copy_ms": copy_ms, "plain_copy_GBps": 2 * nbytes / (copy_ms * 1e-3) / 1e9,
              "bytes_model": "forward reads N*s, backward reads+writes 2*N*s (recompute design, 3*N*s total)"}
    del x, y, g
    torch.cuda.empty_cache()
    return roofline, gather


def pipeline_leg(args, torch, dagx, workloads, dev):
    """Configuration 4 (B=16, L<=1024, T<=256, V=30522, fp16 logits): the criterion's call sequence
    through the public API -- gather (with grad) -> dag_loss fwd+bwd -> gather bwd -- and
    gather (no grad) -> best alignment.  Returns ms per pipeline step."""
    c = workloads.dag_config(4, device=dev)
    g = workloads.gather_config(4, device=dev)
    logits0 = g["logits"]
    Bp, Lp, Vp = logits0.shape
    ol, tl = c["out_len"], c["tgt_len"]
    Tp = c["T"]
    gen = torch.Generator().manual_seed(7)
    targets = torch.randint(0, Vp, (Bp, Tp), generator=gen).to(dev)
    idx = targets.unsqueeze(1).expand(-1, Lp, -1)           # stride-0 over the graph axis, as the criterion passes it
    links = c["links"]
    work = torch.empty_like(logits0)

    class _Output(torch.autograd.Function):   # stands for the layer that produced the logits (a non-leaf, no copy)
        @staticmethod
        def forward(ctx, x):
            return x.detach()

        @staticmethod
        def backward(ctx, gx):
            return gx

    def train_step(transposed=False):
        leaf = work.requires_grad_()
        lk = links.detach().requires_grad_()
        _, sel = dagx.dag_logsoftmax_gather_inplace(_Output.apply(leaf), idx, transposed)
        loss = dagx.dag_loss(sel.transpose(1, 2), lk, ol, tl)
        (-(loss / tl).mean()).backward()

    def align_step():
        with torch.no_grad():
            _, sel = dagx.dag_logsoftmax_gather_inplace(work, idx)
            return dagx.dag_best_alignment(sel.transpose(1, 2), links, ol, tl)

    prev = torch.full((Bp, Lp), 3, dtype=torch.int64, device=dev)

    def glat_step():      # the glancing pass of glat_function (nat_dag_loss.py:239-321) with this library's operators
        with torch.no_grad():
            _, sel, pred = dagx.dag_logsoftmax_gather_argmax(work, idx, True)
            path = dagx.dag_best_alignment(sel.transpose(1, 2), links, ol, tl)
            return dagx.dag_glat_glance(path, targets, pred, prev, tl, 0.5)

    def glat_step_reference_glue():   # the same pass with the reference's tensor operations around the two DAG operators
        with torch.no_grad():
            pred = work.argmax(-1)
            _, sel = dagx.dag_logsoftmax_gather_inplace(work, idx)
            path = dagx.dag_best_alignment(sel.transpose(1, 2), links, ol, tl)
            assigned = path >= 0
            oracle = targets.gather(-1, path.clip(min=0))
            same = ((pred == oracle) & assigned).sum(1)
            keep_prob = ((tl - same) / tl * 0.5).unsqueeze(-1) * assigned.float()
            keep = (torch.rand(prev.shape, device=dev) < keep_prob).bool()
            return prev.masked_fill(keep, 0) + oracle.masked_fill(~keep, 0), path.masked_fill(~keep, -1)

    def timed(fn, n):
        times = []
        for _ in range(n + 1):
            work.requires_grad_(False)
            work.copy_(logits0)                              # the backward leaves the gradient in this buffer
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            start.record(); fn(); stop.record()
            torch.cuda.synchronize()
            times.append(start.elapsed_time(stop))
        return sorted(times[1:])[len(times[1:]) // 2]        # first call is the warm-up
    out = {"workload": f"B={Bp} L<={Lp} T<={Tp} V={Vp} fp16 logits, fp32 links; median of 5 single steps (HIP events, launch overhead included)",
           "train_step_ms": timed(train_step, 5), "align_step_ms": timed(align_step, 5),
           # the gather op storing its result as [B,T,L]: dag_loss reads match with unit stride
           "train_step_btl_storage_ms": timed(lambda: train_step(True), 5),
           # arg max + gather + best alignment + glancing: one pass over the logits and three more launches
           "glat_step_ms": timed(glat_step, 5), "glat_step_with_tensor_op_glue_ms": timed(glat_step_reference_glue, 5)}
    del work, logits0, g, c
    torch.cuda.empty_cache()
    return out


def links_leg(args, torch, nat, lib, stream, dev):
    """dag_multihead_links at B=64 L=512 H=8 fp32 (the link predictor's tail at the headline shape)
    through the C ABI, and the same chain of PyTorch calls as the reference model on the same GPU."""
    Bk, Lk, Hk = 64, 512, 8
    translen = Lk - 1
    gen = torch.Generator(device=dev).manual_seed(3)
    content = torch.randn(Bk, Lk, Lk, Hk, device=dev, generator=gen)
    gates = torch.log_softmax(torch.randn(Bk, Lk, Hk, device=dev, generator=gen), -1)
    vend = torch.full((Bk, Lk), Lk, dtype=torch.int64, device=dev)
    links = torch.empty(Bk, Lk, translen, device=dev); lse = torch.empty(Bk, Lk, Hk, device=dev)
    glinks = torch.randn(Bk, Lk, translen, device=dev, generator=gen); ggates = torch.empty(Bk, Lk, Hk, device=dev)
    work = content.clone()

    def fwd():
        nat.check(lib.dagx_links_fwd(content.data_ptr(), 0, gates.data_ptr(), vend.data_ptr(), Bk, Lk, Hk, translen,
                                     links.data_ptr(), lse.data_ptr(), stream))

    def bwd():   # in place on a scratch copy: timing is value independent
        nat.check(lib.dagx_links_bwd(work.data_ptr(), 0, gates.data_ptr(), vend.data_ptr(), Bk, Lk, Hk, translen,
                                     links.data_ptr(), lse.data_ptr(), glinks.data_ptr(), ggates.data_ptr(), stream))
    n = max(5, min(args.steps, 20))   # (the side legs are event-timed: 20 repetitions are enough)
    fwd_ms = event_time_ms(fwd, n)
    bwd_ms = event_time_ms(bwd, n)
    window = Bk * (Lk * (Lk - 1) // 2) * Hk * 4          # bytes of the allowed (i < j) scores
    out_b = Bk * Lk * translen * 4
    fwd_bytes = window + out_b
    bwd_bytes = window + out_b + Bk * Lk * Lk * Hk * 4
    del work

    # the reference's sequence of calls (glat_decomposed_with_link.py:319-335, 397-404), forward only
    upper = torch.ones(Lk, Lk, dtype=torch.bool, device=dev).triu_(1).unsqueeze(0)
    dst = (torch.arange(Lk, device=dev).unsqueeze(1) + torch.arange(translen, device=dev).unsqueeze(0) + 1).unsqueeze(0)

    def torch_chain():
        c = content.clone()
        mask = upper.expand(Bk, -1, -1)
        res = c.masked_fill_(~mask.unsqueeze(-1), float("-inf")).gather(
            2, dst.clip(max=Lk - 1).unsqueeze(-1).expand(Bk, -1, -1, Hk)).masked_fill_((dst >= Lk).unsqueeze(-1), float("-inf"))
        nouse = ~(mask.any(-1))
        res = res.masked_fill(nouse.unsqueeze(-1).unsqueeze(-1), float("-inf"))
        res = torch.log_softmax(res, dim=2).masked_fill(nouse.unsqueeze(-1).unsqueeze(-1), float("-inf"))
        return torch.logsumexp(res + gates.unsqueeze(2), dim=-1)
    torch_ms = event_time_ms(torch_chain, 3, warmup=1, rounds=1)
    out = {"workload": f"dag_multihead_links B={Bk} L={Lk} H={Hk} fp32, translen={translen}",
           "fwd_ms": fwd_ms, "bwd_ms": bwd_ms,
           "fwd_GBps": fwd_bytes / (fwd_ms * 1e-3) / 1e9, "bwd_GBps": bwd_bytes / (bwd_ms * 1e-3) / 1e9,
           "fwd_frac_of_peak": fwd_bytes / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "bwd_frac_of_peak": bwd_bytes / (bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
           "torch_chain_fwd_ms_same_gpu": torch_ms,
           "bytes_model": "forward reads the allowed scores and writes [B,L,translen]; backward reads the allowed scores "
                          "and grad_links and writes the whole [B,L,L,H] gradient"}
    del content, links, glinks
    torch.cuda.empty_cache()
    return out


def glue_leg(args, torch, dagx, dev):
    """The criterion's glue at B=64 L=512 T=64 (fp32 match): dag_force_alignment forward and
    backward and dag_glat_glance, each one launch, beside the reference's chains of PyTorch calls
    (nat_dag_loss.py:111-120, 273-278 + 307-311) on the same GPU."""
    Bk, Lk, Tk = 64, 512, 64
    gen = torch.Generator(device=dev).manual_seed(4)
    match = torch.randn(Bk, Tk, Lk, device=dev, generator=gen)
    grad = torch.randn(Bk, Tk, Lk, device=dev, generator=gen)
    path = torch.full((Bk, Lk), -1, dtype=torch.int64, device=dev)
    path[:, ::8] = torch.arange(Tk, device=dev)                      # a valid alignment: every 8th node emits
    keep = torch.rand(Bk, Lk, device=dev, generator=gen) < 0.3
    force = path.masked_fill(~keep, -1)
    tgt = torch.randint(4, 40000, (Bk, Tk), device=dev, generator=gen)
    pred = torch.randint(4, 40000, (Bk, Lk), device=dev, generator=gen)
    prev = torch.full((Bk, Lk), 3, dtype=torch.int64, device=dev)
    tgt_len = torch.full((Bk,), Tk, dtype=torch.int64, device=dev)
    rand = torch.rand(Bk, Lk, device=dev, generator=gen)
    pinned = torch.zeros(Bk, Lk, dtype=torch.bool, device=dev)
    from da_transformer_amd.custom_ops.glat import _force_emit

    def torch_force(m):
        hit = torch.zeros(Bk, Tk + 1, Lk, dtype=torch.bool, device=dev).scatter_(1, force.unsqueeze(1) + 1, 1)[:, 1:]
        row = hit.sum(dim=-1, keepdim=True) > 0
        return m.masked_fill(row, 0) + torch.zeros_like(m).masked_fill_(~hit, float("-inf")).masked_fill_(~row, 0)

    def torch_glance():
        assigned = path >= 0
        oracle = tgt.gather(-1, path.clip(min=0))
        same = ((pred == oracle) & assigned & ~pinned).sum(1)
        kp = ((tgt_len - pinned.sum(dim=-1) - same) / tgt_len * 0.5).unsqueeze(-1) * assigned.float()
        kw = (rand < kp).bool() | pinned
        return prev.masked_fill(kw, 0) + oracle.masked_fill(~kw, 0), path.masked_fill(~kw, -1)
    n = max(5, min(args.steps, 20))   # (the side legs are event-timed: 20 repetitions are enough)
    out = {"workload": f"criterion glue B={Bk} L={Lk} T={Tk}, fp32 match",
           "force_alignment_fwd_ms": event_time_ms(lambda: _force_emit(match, force, False), n),
           "force_alignment_bwd_ms": event_time_ms(lambda: _force_emit(grad, force, True), n),
           "glat_glance_ms": event_time_ms(lambda: dagx.dag_glat_glance(path, tgt, pred, prev, tgt_len, 0.5, rand=rand), n),
           "torch_force_alignment_fwd_ms_same_gpu": event_time_ms(lambda: torch_force(match), n),
           "torch_glance_ms_same_gpu": event_time_ms(torch_glance, n),
           "bytes_force_alignment": 2 * Bk * Tk * Lk * 4 + Bk * Lk * 8,
           "note": "times include the output allocations of the Python wrappers; the kernels are at the launch floor"}
    return out


def decode_leg(args, torch, dagx, nat, lib, stream, dev):
    """dag_viterbi_decode (jointviterbi) at B=64 L=512, decode_upsample_scale 8 (128 steps), beside the
    reference's sequence of PyTorch calls and host loops (glat_decomposed_with_link.py:625-626,
    720-777) on the same GPU and host."""
    import time
    Bk, Lk, scale, beta, pad = 64, 512, 8.0, 1.0, 1
    translen = Lk - 1
    max_length = int(2 * Lk / scale)
    gen = torch.Generator(device=dev).manual_seed(6)
    i = torch.arange(Lk, device=dev).view(1, Lk, 1); j = torch.arange(Lk, device=dev).view(1, 1, Lk)
    out_len = torch.randint(128, Lk + 1, (Bk,), device=dev, generator=gen); out_len[0] = Lk
    ok = (j > i) & (j < out_len.view(Bk, 1, 1))
    logits = torch.randn(Bk, Lk, Lk, device=dev, generator=gen) + 8.0 * (j == i + 4)   # transitions favour i -> i+4: long paths win
    square = torch.log_softmax(logits.masked_fill(~ok, float("-inf")).masked_fill(~ok.any(-1, keepdim=True), 0.0), -1)
    square = square.masked_fill(~ok, float("-inf"))
    shifted = dagx.extract_valid_links(square, translen).contiguous()
    u, tok = torch.log_softmax(torch.randn(Bk, Lk, 50, device=dev, generator=gen) * 2, -1).max(-1)
    del logits, ok

    penalty = ((torch.arange(max_length) + 1) ** beta).to(torch.float32).to(dev)
    out_tokens, nodes = torch.empty((2, Bk, max_length), dtype=torch.int64, device=dev).unbind(0)
    out_count, pred_length = torch.empty((2, Bk), dtype=torch.int64, device=dev).unbind(0)
    nbytes = nat.workspace_bytes(nat.OP_VITERBI_DECODE, Bk, max_length, Lk, translen)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)

    def kernels():
        nat.check(lib.dagx_viterbi_decode(shifted.data_ptr(), 0, u.data_ptr(), tok.data_ptr(), out_len.data_ptr(), Bk, Lk, translen,
                                          max_length, penalty.data_ptr(), 1, pad, out_tokens.data_ptr(), out_count.data_ptr(),
                                          pred_length.data_ptr(), nodes.data_ptr(), ws.data_ptr(), nbytes, stream))
    n = max(5, min(args.steps, 20))   # (the side legs are event-timed: 20 repetitions are enough)
    kernels_ms = event_time_ms(kernels, n)

    def wall_ms(fn, reps):
        fn(); torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / reps * 1e3
    ours = lambda: dagx.dag_viterbi_decode(shifted, (u, tok), out_len, scale, beta, True, pad)
    ours_wall_ms = wall_ms(ours, n)

    def reference_chain():
        links = dagx.restore_valid_links(shifted)                 # :625-626
        tokens = tok.tolist()
        reach = links[:, 0]
        reach += u[:, 0].unsqueeze(1)
        reach += u
        per_step, back = [reach], []
        for _ in range(max_length - 1):
            reach, source = torch.max(reach.unsqueeze(-1) + links, dim=1)
            reach += u
            per_step.append(reach); back.append(source)
        back = torch.stack(back, dim=0); per_step = torch.stack(per_step, dim=0)
        per_step += torch.gather(links, -1, (out_len - 1).view(Bk, 1, 1).repeat(1, Lk, 1)).view(1, Bk, Lk)
        best, last_node = torch.max(per_step, dim=-1)
        lengths = torch.arange(max_length).unsqueeze(-1).repeat(1, Bk) + 1
        best = best / (lengths ** beta).to(dev)
        _, n_pred = torch.max(best, dim=0)
        n_pred = n_pred + 1
        start = torch.gather(last_node, 0, (n_pred - 1).view(1, Bk)).view(Bk).tolist()
        back = back.tolist()
        out = []
        for b, cnt in enumerate(n_pred.tolist()):
            node = start[b]; seen = tokens[b][node]; res = [seen]
            for k in range(cnt - 1):
                node = back[cnt - k - 2][b][node]
                t = tokens[b][node]
                if t != pad and t != seen:
                    res.insert(0, t)
                seen = t
            out.append(res)
        longest = max(len(r) for r in out)
        return torch.tensor([r + [pad] * (longest - len(r)) for r in out])
    ref_wall_ms = wall_ms(reference_chain, 2)
    same = bool(torch.equal(ours().output_tokens, reference_chain()))
    # greedy walk (decode_strategy lookahead, decode_beta 1), :691-718
    la_tokens, la_nodes = torch.empty((2, Bk, Lk), dtype=torch.int64, device=dev).unbind(0)
    la_count = torch.empty(Bk, dtype=torch.int64, device=dev)

    def lookahead_kernel():
        nat.check(lib.dagx_lookahead_decode(shifted.data_ptr(), 0, u.data_ptr(), tok.data_ptr(), out_len.data_ptr(), Bk, Lk, translen,
                                            1.0, 0, pad, la_tokens.data_ptr(), la_count.data_ptr(), la_nodes.data_ptr(), stream))
    lookahead_ms = event_time_ms(lookahead_kernel, n)
    la_ours = lambda: dagx.dag_lookahead_decode(shifted, (u, tok), out_len, 1.0, False, pad)
    la_wall_ms = wall_ms(la_ours, n)

    def lookahead_reference_chain():
        links = dagx.restore_valid_links(shifted)
        tokens = tok.tolist()
        lengths = out_len.cpu().tolist()
        successor = (links + u.unsqueeze(1) * 1.0).max(dim=-1)[1].cpu().tolist()
        out = []
        for b, length in enumerate(lengths):
            seen = tokens[b][0]; node = 0; res = [seen]
            while node != length - 1:
                node = successor[b][node]
                t = tokens[b][node]
                if t != pad and t != seen:
                    res.append(t)
                seen = t
            out.append(res)
        longest = max(len(r) for r in out)
        return torch.tensor([r + [pad] * (longest - len(r)) for r in out])
    la_ref_ms = wall_ms(lookahead_reference_chain, 3)
    la_same = bool(torch.equal(la_ours().output_tokens, lookahead_reference_chain()))
    pairs = Bk * (max_length - 1) * (Lk * (Lk - 1) // 2)
    out = {"workload": f"viterbi decoding (jointviterbi) B={Bk} L={Lk} steps={max_length} fp32 links, beta={beta}",
           "lookahead": {"kernel_ms": lookahead_ms, "end_to_end_wall_ms": la_wall_ms,
                         "reference_torch_chain_wall_ms_same_gpu": la_ref_ms, "tokens_equal_to_reference_chain_on_gpu": la_same,
                         "GBps": Bk * Lk * translen * 4 / (lookahead_ms * 1e-3) / 1e9},
           "kernels_ms": kernels_ms, "end_to_end_wall_ms": ours_wall_ms,
           "reference_torch_chain_wall_ms_same_gpu": ref_wall_ms,
           "tokens_equal_to_reference_chain_on_gpu": same,
           "pair_updates_upper_bound": pairs, "pair_updates_per_s": pairs / (kernels_ms * 1e-3),
           "mean_pred_length": float(pred_length.float().mean())}
    del square, shifted, ws
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (a step is 0.18 ms: with few timed steps the one-off latency of the first launch and of the closing
    #  synchronisation, about 0.2 ms together, shows in the per-step figure -- 0.188 ms at 20 steps, 0.178 at 400)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--skip-cpu", action="store_true", help="skip the host-core baseline leg")
    ap.add_argument("--skip-gather", action="store_true", help="skip the [64,512,40000] gather leg")
    ap.add_argument("--leg", choices=["all", "dag", "dag-headline", "gather", "links", "glue", "decode", "pipeline"], default="all",
                    help="profiling aid: run one part only (the JSON line is then partial); dag-headline launches nothing but "
                         "the headline shape's DAG-loss and alignment kernels, so that per-kernel profile rows are that shape's")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (the operators are per-sample and never "
                 "communicate); --gpus must be 1")

    import torch
    import da_transformer_amd as dagx
    from da_transformer_amd import _native as nat
    import workloads

    if not torch.cuda.is_available():
        sys.exit("bench.py: needs a GPU")
    dev = "cuda:0"
    torch.cuda.set_device(0)
    lib = nat.lib()
    stream = torch.cuda.current_stream().cuda_stream

    if args.leg == "links":
        print(json.dumps({"leg": "links", "multihead_links": links_leg(args, torch, nat, lib, stream, dev)}))
        return
    if args.leg == "pipeline":
        print(json.dumps({"leg": "pipeline", "pipeline_cfg4": pipeline_leg(args, torch, dagx, workloads, dev)}))
        return
    if args.leg == "decode":
        print(json.dumps({"leg": "decode", "viterbi_decode": decode_leg(args, torch, dagx, nat, lib, stream, dev)}))
        return
    if args.leg == "glue":
        print(json.dumps({"leg": "glue", "criterion_glue": glue_leg(args, torch, dagx, dev)}))
        return
    if args.leg == "gather":
        print(json.dumps({"leg": "gather", "logsoftmax_gather": gather_leg(args, torch, nat, lib, stream, workloads, dev)[1]}))
        return

    # ------------------------------------------------------------------ headline: dag_loss fwd+bwd
    cfg = workloads.dag_config(1, device=dev, rect=True)          # fp16 inputs, B=64 L=512 T=64
    B, T, L = cfg["B"], cfg["T"], cfg["L"]
    match16, links16 = cfg["match"], cfg["links"]
    ol, tl, gout = cfg["out_len"], cfg["tgt_len"], cfg["grad_out"]
    translen = links16.shape[2]
    U = pair_updates(ol.cpu(), tl.cpu(), translen)

    def api_step(match, links):
        m = match.detach().requires_grad_()
        lk = links.detach().requires_grad_()
        loss = dagx.dag_loss(m, lk, ol, tl)
        loss.backward(gout)
        return loss, m.grad, lk.grad

    def headline():
        """W untimed steps, then exactly K timed ones between two synchronisations."""
        for _ in range(args.warmup):
            api_step(match16, links16)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            api_step(match16, links16)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return wall * 1e3 / args.steps, B * args.steps / wall

    # kernel-level timing through the C ABI, buffers preallocated
    def dag_kernel_times(match, links, ol=ol, tl=tl, gout=gout):
        B, T, L = match.shape
        translen = links.shape[2]
        nblk = (L + 63) // 64
        hats = torch.empty(2, B, T, L, device=dev); offs = torch.empty(2, B, T, nblk, dtype=torch.float64, device=dev)
        logz = torch.empty(2, B, dtype=torch.float64, device=dev); loss = torch.empty(B, device=dev)
        gm = torch.empty(B, T, L, dtype=match.dtype, device=dev); gl = torch.empty_like(links)
        flags = torch.empty(B, dtype=torch.int32, device=dev)
        ms3 = nat.strides3(match)
        mdt, ldt = nat.dtype_code(match), nat.dtype_code(links)
        nb_f = nat.workspace_bytes(nat.OP_LOSS_FWD, B, T, L, translen)
        ws = torch.zeros(max(nb_f, 4), dtype=torch.uint8, device=dev)   # the forward wants it zero and leaves it zero

        def fwd(need_grad=1):
            nat.check(lib.dagx_loss_fwd(match.data_ptr(), mdt, ms3, links.data_ptr(), ldt, ol.data_ptr(), tl.data_ptr(),
                                        B, T, L, translen, hats[0].data_ptr(), hats[1].data_ptr(), offs[0].data_ptr(),
                                        offs[1].data_ptr(), logz.data_ptr(), loss.data_ptr(), flags.data_ptr(), need_grad,
                                        ws.data_ptr(), nb_f, stream))

        def bwd(with_match=True):
            nat.check(lib.dagx_loss_bwd(gout.data_ptr(), 1, hats[0].data_ptr(), hats[1].data_ptr(), offs[0].data_ptr(),
                                        offs[1].data_ptr(), logz.data_ptr(), flags.data_ptr(), match.data_ptr(), mdt, ms3,
                                        links.data_ptr(), ldt, ol.data_ptr(), tl.data_ptr(), B, T, L, translen,
                                        gm.data_ptr() if with_match else None, gl.data_ptr(), None, 0, stream))

        n = max(5, min(args.steps, 20))   # (the side legs are event-timed: 20 repetitions are enough)
        out = dict(fwd_ms=event_time_ms(fwd, n), bwd_ms=event_time_ms(bwd, n),
                   grad_links_ms=event_time_ms(lambda: bwd(False), n),
                   fwd_no_grad_ms=event_time_ms(lambda: fwd(0), n))
        fwd()
        out["samples_settled_by_float64_tile_sweeps"] = int((flags == 2).sum().item())
        out["samples_redone_by_log_domain_kernel"] = int((flags == 1).sum().item())
        u = pair_updates(ol.cpu(), tl.cpu(), translen)
        out["pair_updates_fwd_bwd"] = 3 * u
        out["frac_of_valu_peak"] = 3 * u / ((out["fwd_ms"] + out["bwd_ms"]) * 1e-3) / VALU_PEAK_LANEOPS
        return out

    k16 = dag_kernel_times(match16, links16)
    match32, links32 = match16.float(), links16.float()
    k32 = None if args.leg == "dag-headline" else dag_kernel_times(match32, links32)
    api32_ms = None
    if args.leg != "dag-headline":
        for _ in range(2):
            api_step(match32, links32)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(max(5, min(args.steps, 200) // 2)):
            api_step(match32, links32)
        torch.cuda.synchronize()
        api32_ms = (time.perf_counter() - t0) * 1e3 / max(5, min(args.steps, 200) // 2)

    # alignment (fp32 inputs, configuration 3 at the rectangular shape)
    path = torch.empty(B, L, dtype=torch.int64, device=dev)
    nb_a = nat.workspace_bytes(nat.OP_BEST_ALIGNMENT, B, T, L, translen)
    ws_a = torch.empty(max(nb_a, 1), dtype=torch.uint8, device=dev)

    def align():
        nat.check(lib.dagx_best_alignment(match32.data_ptr(), nat.F32, nat.strides3(match32), links32.data_ptr(), nat.F32,
                                          ol.data_ptr(), tl.data_ptr(), B, T, L, translen, path.data_ptr(),
                                          ws_a.data_ptr(), nb_a, stream))
    align_ms = event_time_ms(align, max(5, min(args.steps, 50)))

    # The headline loop runs here, behind the kernel-level legs of the same shape: with few warm-up steps right after
    # start-up the device is still raising its clocks and the caching allocator still growing (5 timed steps behind
    # 1 warm-up step: 0.27 ms / step there).
    ms_per_step, value = headline()

    if args.leg == "dag-headline":
        # (the roofline object as in the full line; then the calibration copies for the HBM byte counters)
        fwd_s = k16["fwd_ms"] * 1e-3
        calib_src = torch.empty(CALIBRATION_COPY_BYTES, dtype=torch.uint8, device=dev).fill_(1)
        calib_dst = torch.empty_like(calib_src)
        for _ in range(3):
            calib_dst.copy_(calib_src)
        torch.cuda.synchronize()
        print(json.dumps({"leg": "dag-headline", "calibration_copy_bytes": CALIBRATION_COPY_BYTES, "ms_per_step": ms_per_step,
                          "samples_per_s": value, "dag_kernels_fp16_in_ms": k16, "best_alignment_fp32_ms": align_ms,
                          "sweep_frac_of_valu_peak": 2 * U / fwd_s / VALU_PEAK_LANEOPS}))
        return

    # torch-native path on the same GPU (public torch_* functions of the package, square links)
    sq = dagx.restore_valid_links(links32)

    def torch_gpu_step():
        m = match32.detach().requires_grad_()
        s = sq.detach().requires_grad_()
        loss = dagx.torch_dag_loss(m, s, ol, tl)
        loss.backward(gout)
    torch_gpu_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n_t = 3
    for _ in range(n_t):
        torch_gpu_step()
    torch.cuda.synchronize()
    torch_gpu_ms = (time.perf_counter() - t0) * 1e3 / n_t
    del sq
    torch.cuda.empty_cache()

    # ---- roofline of the headline's dominant kernel: the tile sweeps (one launch = both sweeps = 2U pair-updates;
    #      the timed forward also contains the check launch behind it, which finds nothing to redo) ----
    fwd_s = k16["fwd_ms"] * 1e-3
    sweep_traffic = traffic_bytes("dag_loss_B64_L512_T64_hbm_traffic.md", "dagx::dag_sweep_tiles_kernel<__half, __half, false>", 3, 4)
    # LDS and vector-ALU utilisation of the same kernel from the committed counter summary (profiles/): busy fractions
    # of the LDS pipeline (128 bytes per clock and CU) and of the SIMDs, and the source revision they were taken at
    lds_row = profile_table_row("dag_loss_B64_L512_T64_sq_counters.md", "dagx::dag_sweep_tiles_kernel<__half, __half, false>")
    def cell_frac(cells, col):
        try:
            return float(cells[col].rstrip("%")) / 100.0
        except (TypeError, ValueError, IndexError):
            return None
    trace_row = profile_table_row("dag_loss_B64_L512_T64_kernel_trace.md", "dagx::dag_sweep_tiles_kernel<__half, __half, false>")
    try:
        trace_avg_us = float(trace_row[2])
    except (TypeError, ValueError, IndexError):
        trace_avg_us = None
    roofline = {"kernel": "dag_sweep_tiles_kernel<half,half,float32 numbers> (dagx_loss_fwd: the sweeps of alpha and beta)",
                "valu_busy_frac": cell_frac(lds_row, 4), "lds_frac": cell_frac(lds_row, 8), "lds_bank_conflict_frac": cell_frac(lds_row, 9),
                "counters_from": profile_source_revision("dag_loss_B64_L512_T64_sq_counters.md"),
                "bound": "valu", "achieved": 2 * U / fwd_s, "peak": VALU_PEAK_LANEOPS, "unit": "pair-updates/s",
                "frac": 2 * U / fwd_s / VALU_PEAK_LANEOPS, "traffic": sweep_traffic,
                "algorithmic_pair_updates": 2 * U, "kernel_ms": k16["fwd_ms"],
                # kernel_ms is one dagx_loss_fwd between HIP events: the float32 tile sweeps and, behind them, the float64 and
                # log-domain launches, idle here (4.6 us each in a kernel trace, about 1 us each back to back); the
                # committed kernel trace has the tile kernel by itself
                "kernel_ms_covers": "float32 tile sweeps + the idle float64 and log-domain launches of the same call",
                "kernel_alone_avg_us_in_profile": trace_avg_us,
                "frac_kernel_alone_from_profile": (2 * U / (trace_avg_us * 1e-6) / VALU_PEAK_LANEOPS) if trace_avg_us else None,
                "achieved_TFLOPs": 2 * 2 * U / fwd_s / 1e12,
                "frac_of_published_fp32_vector_peak": 2 * 2 * U / fwd_s / 157.3e12,
                "note": "peak = 256 CUs x 64 fp32 lanes x 2.4 GHz, one FMA per pair-update (the published 157.3 TFLOP/s "
                        "counts packed FMAs, which this build does not use); traffic = HBM bytes per launch (not the bound)"}
    dp_time_s = (k16["fwd_ms"] + k16["bwd_ms"]) * 1e-3
    roofline_dp = {"bound": "valu", "achieved": 3 * U / dp_time_s, "peak": VALU_PEAK_LANEOPS,
                   "unit": "pair-updates/s", "frac": 3 * U / dp_time_s / VALU_PEAK_LANEOPS,
                   "pair_updates_per_step": 3 * U, "kernel_ms": dp_time_s * 1e3,
                   # the same work against the timed steps themselves (forward and backward alternate there, so a
                   # launch is set up while its predecessor drains; the legs above time each on its own)
                   "timed_step_ms": ms_per_step, "frac_over_timed_steps": 3 * U / (ms_per_step * 1e-3) / VALU_PEAK_LANEOPS}

    # ---- other DAG-loss workloads (kernel times through the C ABI) ----
    def other_dag_legs():
        out = {}
        c = workloads.dag_config(1, device=dev)                      # ragged lengths as drawn (8 * U{16..64} nodes, U{16..64} targets)
        out["ragged_cfg1_fp16"] = dict(workload="B=64 L<=512 T<=64 drawn lengths, fp16",
                                       **dag_kernel_times(c["match"], c["links"], c["out_len"], c["tgt_len"], c["grad_out"]))
        # the shape of the reference's own self-check and tuner (fs_plugins/custom_ops/dag_loss.py:384-398, 528-533)
        gen = torch.Generator(device=dev).manual_seed(50)
        tarlen = 50; bsz = 4096 // tarlen; prelen = 8 * tarlen
        m = torch.rand(bsz, tarlen, prelen, device=dev, generator=gen)
        lk = torch.rand(bsz, prelen, 32, device=dev, generator=gen).log_softmax(-1)
        o = prelen - torch.randint(0, 5, (bsz,), device=dev, generator=gen)
        t = tarlen - torch.randint(0, 5, (bsz,), device=dev, generator=gen)
        g = torch.full((bsz,), 1.0 / bsz, device=dev)
        out["reference_tuner_shape_fp32"] = dict(workload=f"B={bsz} L={prelen} T={tarlen} translen=32 fp32, lengths shortened by 0..4",
                                                 **dag_kernel_times(m, lk, o, t, g))
        # larger batches at the headline shape (the reference's own tuner runs bsz = 4096 // tarlen ~ 80,
        # fs_plugins/custom_ops/dag_loss.py:528-533): more workgroups than the 256 CUs hold at once
        for bsz in (128, 256):
            c = workloads.dag_config(1, device=dev, rect=True, B=bsz)
            k = dag_kernel_times(c["match"], c["links"], c["out_len"], c["tgt_len"], c["grad_out"])
            k["samples_per_s_fwd_bwd"] = bsz / ((k["fwd_ms"] + k["bwd_ms"]) * 1e-3)
            out[f"batch_{bsz}_fp16"] = dict(workload=f"B={bsz} L=512 T=64 all samples full length, fp16", **k)
            del c
        # inputs like a trained model's: what the float32 tile sweeps cannot hold goes to the float64 ones, then to the
        # log-domain kernel; `float64_first` = the same call with dagx_loss_float64_first(1), i.e. without the float32 pass
        for name, (bsz, L_, T_, scale, std) in (("peaked_links_x10_fp32", (64, 512, 64, 10.0, 5.0)),
                                                ("peaked_links_x30_fp32", (64, 512, 64, 30.0, 10.0)),
                                                ("peaked_links_x10_L1024_T256_fp32", (16, 1024, 256, 10.0, 5.0))):
            c = workloads.peaked_config(7, bsz, L_, T_, scale, std, device=dev)
            k = dag_kernel_times(c["match"], c["links"], c["out_len"], c["tgt_len"], c["grad_out"])
            before = lib.dagx_loss_float64_first(1)
            try:
                k64 = dag_kernel_times(c["match"], c["links"], c["out_len"], c["tgt_len"], c["grad_out"])
            finally:
                lib.dagx_loss_float64_first(before)
            k["float64_first"] = {q: k64[q] for q in ("fwd_ms", "fwd_no_grad_ms", "samples_settled_by_float64_tile_sweeps",
                                                      "samples_redone_by_log_domain_kernel")}
            out[name] = dict(workload=f"B={bsz} L<={L_} T<={T_}, transition logits N(0,1)*{scale:g}, token logits std {std:g}, "
                                      "pinned nodes, fp32", **k)
            del c
        return out
    more_dag = other_dag_legs()

    # ---- the float64 operators at the headline shape: float64 arithmetic throughout, kernels of their own, for
    #      checking rather than for speed (the reference's instantiation for double, fs_plugins/custom_ops/dag_loss.cu:160) ----
    def float64_leg():
        m = match16.double().requires_grad_(); lk = links16.double().requires_grad_(); g = gout.double()

        def fwd_bwd():
            m.grad = None; lk.grad = None
            dagx.dag_loss(m, lk, ol, tl).backward(g)

        def fwd_only():
            with torch.no_grad():
                dagx.dag_loss(m, lk, ol, tl)
        return {"workload": "B=64 L=512 T=64 float64 tensors through the public API",
                "dag_loss_fwd_bwd_ms": event_time_ms(fwd_bwd, 3, warmup=1, rounds=1),
                "dag_loss_fwd_no_grad_ms": event_time_ms(fwd_only, 3, warmup=1, rounds=1),
                "best_alignment_ms": event_time_ms(lambda: dagx.dag_best_alignment(m, lk, ol, tl), 3, warmup=1, rounds=1)}
    float64_out = float64_leg() if args.leg == "all" else None

    if args.leg == "dag":
        # plain device copies of a known size: the calibration dispatches for the HBM byte counters
        # (FETCH_SIZE / WRITE_SIZE of a rocprofv3 --pmc run of this leg are scaled by what they read here)
        calib_src = torch.empty(CALIBRATION_COPY_BYTES, dtype=torch.uint8, device=dev).fill_(1)
        calib_dst = torch.empty_like(calib_src)
        for _ in range(3):
            calib_dst.copy_(calib_src)
        torch.cuda.synchronize()
        print(json.dumps({"leg": "dag", "calibration_copy_bytes": CALIBRATION_COPY_BYTES, "ms_per_step": ms_per_step, "dag_kernels_fp16_in_ms": k16,
                          "dag_kernels_fp32_in_ms": k32, "roofline": roofline, "roofline_dp": roofline_dp,
                          "dag_other_workloads": more_dag}))
        return

    # ------------------------------------------------------------------ gather leg (configuration 2)
    roofline_gather, gather = (None, None) if args.skip_gather else gather_leg(args, torch, nat, lib, stream, workloads, dev)
    pipeline = None if args.skip_gather else pipeline_leg(args, torch, dagx, workloads, dev)
    links_out = None if args.skip_gather else links_leg(args, torch, nat, lib, stream, dev)
    glue_out = glue_leg(args, torch, dagx, dev)
    decode_out = None if args.skip_gather else decode_leg(args, torch, dagx, nat, lib, stream, dev)

    # ------------------------------------------------------------------ host-core baseline (torch-native CPU)
    cpu_baseline = None
    if not args.skip_cpu:
        from oracle import torch_native as tn
        nb = 16          # with the repetitions below about 10 s of work on the box's 16 host cores
        torch.set_num_threads(os.cpu_count() or 1)
        m_cpu = match16[:nb].float().cpu(); l_cpu = tn.restore_valid_links(links16[:nb].float().cpu())
        ol_c, tl_c, g_c = ol[:nb].cpu(), tl[:nb].cpu(), gout[:nb].cpu()

        def cpu_step():
            m = m_cpu.clone().requires_grad_(); s = l_cpu.clone().requires_grad_()
            tn.torch_dag_loss(m, s, ol_c, tl_c).backward(g_c)
        cpu_step()
        reps = 30
        t0 = time.perf_counter()
        for _ in range(reps):
            cpu_step()
        cpu_s = (time.perf_counter() - t0) / reps
        cpu_baseline = {"value": nb / cpu_s, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
                        "sample": f"torch-native dag_loss fwd+bwd, fp32, {nb} samples of the headline shape "
                                  f"(L=512, T=64), {reps} timed repetitions"}

    out = {
        "metric": "DAG-loss fwd+bwd samples/sec @B64,L512,T64; logsoftmax_gather HBM GB/s",
        "value": value, "unit": "samples/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "dag_loss fwd+bwd, B=64 L=512 T=64 all samples full length, translen=511, "
                               "fp16 match/links with fp32 accumulation (public Python API incl. autograd)"},
        "roofline": roofline,
        "roofline_dp": roofline_dp,
        "roofline_gather": roofline_gather,
        "dag_other_workloads": more_dag,
        "cpu_baseline": cpu_baseline,
        "dag_kernels_fp16_in_ms": k16, "dag_kernels_fp32_in_ms": k32,
        "dag_api_fp32_in_ms_per_step": api32_ms,
        "best_alignment_ms": align_ms,
        "float64_operators": float64_out,
        "torch_native_same_gpu_ms_per_step": torch_gpu_ms,
        "speedup_vs_torch_native_same_gpu": torch_gpu_ms / ms_per_step,
        "logsoftmax_gather": gather,
        "pipeline_cfg4": pipeline,
        "multihead_links": links_out,
        "criterion_glue": glue_out,
        "viterbi_decode": decode_out,
        "device": torch.cuda.get_device_name(0),
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
