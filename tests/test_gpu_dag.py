"""GPU parity of dag_loss / dag_best_alignment (through the C ABI) against the CPU oracle."""
import math
import os

import numpy as np
import pytest
import torch

import da_transformer_amd as dagx
from conftest import ROOT
from oracle import cref
from oracle import torch_native as tn
from helpers import random_problem, path_nodes, NEG_INF
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def hip_loss_and_grads(match, links, ol, tl, g=None):
    m = match.to(DEV).requires_grad_()
    lk = links.to(DEV).requires_grad_()
    loss = dagx.dag_loss(m, lk, ol.to(DEV), tl.to(DEV))
    if g is None:
        g = torch.ones(loss.shape[0])
    fin = torch.isfinite(loss)
    (loss.masked_fill(~fin, 0) * g.to(DEV)).sum().backward()
    return loss.detach().cpu(), m.grad.cpu(), lk.grad.cpu()


def oracle_loss_and_grads(match, links_shifted, ol, tl, g=None):
    """float64 C oracle on the upcast inputs; grad_links returned in the shifted layout."""
    B = match.shape[0]
    g = torch.ones(B) if g is None else g
    sq = tn.restore_valid_links(links_shifted.double())
    loss, gm, gl = cref.dag_loss_grad(match.double().numpy(), sq.numpy(), ol.numpy(), tl.numpy(), g.double().numpy())
    gl = tn.extract_valid_links(torch.from_numpy(gl), links_shifted.shape[2])
    gl = gl.masked_fill(torch.isinf(gl), 0.0)
    return torch.from_numpy(loss), torch.from_numpy(gm), gl


def assert_close(got, ref, rtol, what):
    ref = ref.double(); got = got.double()
    fin = torch.isfinite(ref)
    assert torch.equal(torch.isfinite(got), fin), what
    atol = rtol * ref[fin].abs().max().item() if fin.any() else 0.0
    err = (got[fin] - ref[fin]).abs()
    bound = atol + rtol * ref[fin].abs()
    assert (err <= bound).all(), f"{what}: max err {err.max().item():.3e} (atol {atol:.3e})"


@pytest.mark.parametrize("name", ["dag_cfg0.npz", "dag_cfg0_ragged_translen20.npz"])
def test_golden_fixtures(name):
    z = np.load(os.path.join(ROOT, "tests", "golden", name))
    t = {k: torch.from_numpy(z[k]) for k in z.files}
    loss, gm, gl = hip_loss_and_grads(t["match"], t["links"], t["out_len"], t["tgt_len"], t["grad_out"])
    assert_close(loss, t["loss"], 1e-4, "loss")
    assert_close(gm, t["grad_match"], 1e-4, "grad_match")
    assert_close(gl, t["grad_links"], 1e-4, "grad_links")
    path = dagx.dag_best_alignment(t["match"].to(DEV), t["links"].to(DEV), t["out_len"].to(DEV), t["tgt_len"].to(DEV))
    assert path.dtype == torch.int64 and torch.equal(path.cpu(), t["path"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("translen", [None, 32, 5])
def test_loss_and_grads_ragged(dtype, translen):
    B, L, T = 6, 150, 40
    match, links_sq, ol, tl = random_problem(77, B, L, T, dtype=torch.float32, translen=translen)
    ol[0], tl[0] = L, T
    ol[1], tl[1] = 70, 2
    ol[2], tl[2] = 40, 23
    match = match.to(dtype); links = tn.extract_valid_links(links_sq, translen).to(dtype)
    g = torch.randn(B, generator=torch.Generator().manual_seed(1))
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    rtol = RTOL[dtype]
    assert loss.dtype == torch.float32 and gm.dtype == dtype and gl.dtype == dtype
    assert_close(loss, rloss, 1e-4, "loss")   # accumulation is fp32 whatever the input dtype
    assert_close(gm.float(), rgm, rtol, "grad_match")
    assert_close(gl.float(), rgl, rtol, "grad_links")
    # padding receives exactly zero
    for b in range(B):
        assert (gm[b, int(tl[b]):] == 0).all() and (gm[b, :, int(ol[b]):] == 0).all()
        assert (gl[b, int(ol[b]) - 1:] == 0).all()


def test_strided_match_view_and_no_grad_path():
    """match arrives as the transpose of the gather output ([B,L,T] memory) in the criterion."""
    B, L, T = 3, 65, 9
    match, links_sq, ol, tl = random_problem(3, B, L, T, dtype=torch.float32)
    links = tn.extract_valid_links(links_sq)
    mt = match.transpose(1, 2).contiguous().to(DEV)          # [B,L,T] memory
    view = mt.transpose(1, 2)                                # logical [B,T,L], not contiguous
    with torch.no_grad():
        l1 = dagx.dag_loss(view, links.to(DEV), ol.to(DEV), tl.to(DEV))
    l2, _, _ = hip_loss_and_grads(match, links, ol, tl)
    rloss, _, _ = oracle_loss_and_grads(match, links, ol, tl)
    assert_close(l1.cpu(), rloss, 1e-4, "loss (alpha read-out, strided)")
    assert_close(l2, rloss, 1e-4, "loss (beta read-out)")
    v = view.detach().requires_grad_()
    dagx.dag_loss(v, links.to(DEV), ol.to(DEV), tl.to(DEV)).sum().backward()
    _, rgm, _ = oracle_loss_and_grads(match, links, ol, tl)
    assert_close(v.grad.cpu(), rgm, 1e-4, "grad through a strided view")


def test_infeasible_and_masked_samples():
    B, L, T = 5, 40, 8
    match, links_sq, ol, tl = random_problem(11, B, L, T, dtype=torch.float32, ragged=False)
    links = tn.extract_valid_links(links_sq)
    links[0, 0, :] = NEG_INF                   # node 0 has no way out
    ol[1], tl[1] = 5, 8                        # target longer than the graph
    force = torch.full((B, L), -1, dtype=torch.long); force[2, 17] = 3
    match = tn.force_alignment(match, force)   # -inf inside match
    ol[3], tl[3] = 2, 2                        # smallest legal sample
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert loss[0] == -math.inf and loss[1] == -math.inf
    assert (gm[0] == 0).all() and (gl[0] == 0).all() and (gm[1] == 0).all() and (gl[1] == 0).all()
    assert not torch.isnan(gm).any() and not torch.isnan(gl).any()
    keep = [2, 3, 4]
    rloss, rgm, rgl = oracle_loss_and_grads(match[keep], links[keep], ol[keep], tl[keep])
    assert_close(loss[keep], rloss, 1e-4, "loss")
    assert_close(gm[keep], rgm, 1e-4, "grad_match")
    assert_close(gl[keep], rgl, 1e-4, "grad_links")
    # the pinned target is emitted by node 17 with posterior exactly 1, by no other node
    assert abs(gm[2, 3, 17].item() - 1.0) < 1e-4 and gm[2, 3].abs().sum().item() == pytest.approx(gm[2, 3, 17].item())
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert (path[0] == -1).all() and (path[1] == -1).all()
    assert path[2, 17] == 3 and path_nodes(path[3]) == [0, 1]


def _torch_path(match, links_shifted, ol, tl):
    return tn.torch_dag_best_alignment(match.float(), tn.restore_valid_links(links_shifted.float()), ol, tl)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("translen", [None, 32])
def test_alignment_bit_exact(dtype, translen):
    B, L, T = 8, 200, 31
    match, links_sq, ol, tl = random_problem(123, B, L, T, dtype=torch.float32, translen=translen)
    if translen is not None:                   # keep a path possible: (T_b-1)*translen+1 >= L_b
        ol = torch.minimum(ol, (tl - 1) * translen + 1)
    match = match.to(dtype); links = tn.extract_valid_links(links_sq, translen).to(dtype)
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV))
    assert path.shape == (B, L) and path.dtype == torch.int64 and not path.requires_grad
    assert torch.equal(path.cpu(), _torch_path(match, links, ol, tl))


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_alignment_ties_lowest_index(mode):
    """Exact ties, by the tile kernels (0) and by the one-workgroup method (1: as a launch of its own, 2: inside the
    backtrack launch), whose lanes share a node's predecessors and must still agree on the lowest index."""
    from da_transformer_amd import _native as nat
    before = nat.lib().dagx_force_log_domain(mode)
    try:
        B, L, T = 3, 70, 12
        ol = torch.tensor([70, 33, 12]); tl = torch.tensor([12, 5, 12])
        match = torch.zeros(B, T, L)
        links = workloads.make_links_shifted(torch.Generator().manual_seed(0), ol, L, "cpu")
        links = torch.zeros_like(links).masked_fill(torch.isinf(links), NEG_INF)       # all finite links 0
        path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
        for b in range(B):
            assert path_nodes(path[b]) == list(range(int(tl[b]) - 1)) + [int(ol[b]) - 1]
        # heavily quantised random values: many exact ties, must still equal the torch rule
        for seed, B, L, T in ((9, 6, 90, 17), (10, 3, 400, 33)):
            match, links_sq, ol, tl = random_problem(seed, B, L, T, dtype=torch.float32)
            match = (match * 2).round() / 2
            links = tn.extract_valid_links(links_sq)
            links = ((links * 2).round() / 2).masked_fill(torch.isinf(links), NEG_INF)
            path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
            assert torch.equal(path, _torch_path(match, links, ol, tl))
    finally:
        nat.lib().dagx_force_log_domain(before)


def test_headline_shape_properties_and_sample_parity():
    """B=64, L=512, T=64 (ragged lengths, fp32, fp16 and bf16 inputs): every sample against the float64 C oracle and
    through the invariants, every alignment against the lowest-index rule."""
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        c = workloads.dag_config(3, device=DEV, dtype=dtype)
        if dtype != torch.float32:
            # fp16 gradients of magnitude 1e-6 would be subnormal; scale like a loss scaler does
            c["grad_out"] = c["grad_out"] * 1024
        m = c["match"].requires_grad_(); lk = c["links"].requires_grad_()
        loss = dagx.dag_loss(m, lk, c["out_len"], c["tgt_len"])
        (loss * c["grad_out"]).sum().backward()
        ol, tl, g = c["out_len"].cpu(), c["tgt_len"].cpu(), c["grad_out"].cpu().double()
        gm, gl = m.grad.double().cpu(), lk.grad.double().cpu()
        tol = {torch.float32: 2e-3, torch.float16: 2e-2, torch.bfloat16: 8e-2}[dtype]   # (a bf16 gradient carries 8 bits)
        for b in range(c["B"]):
            Tb = int(tl[b])
            node_mass = gm[b, :Tb].sum(-1) / g[b]
            assert (node_mass - 1).abs().max() < tol, (b, node_mass)
            assert abs(gl[b].sum().item() / g[b].item() - (Tb - 1)) < tol * Tb
            assert (gm[b, Tb:] == 0).all() and (gm[b, :, int(ol[b]):] == 0).all()
        pick = list(range(c["B"]))
        rloss, rgm, rgl = oracle_loss_and_grads(c["match"].detach().cpu()[pick], c["links"].detach().cpu()[pick],
                                                ol[pick], tl[pick], g[pick].float())
        rtol = RTOL[dtype]
        assert_close(loss.detach().cpu()[pick], rloss, 1e-4, "loss")
        assert_close(gm[pick], rgm, rtol, "grad_match")
        assert_close(gl[pick], rgl, rtol, "grad_links")
        with torch.no_grad():
            path = dagx.dag_best_alignment(c["match"].detach(), c["links"].detach(), c["out_len"], c["tgt_len"]).cpu()
        ref, _ = cref.best_alignment(c["match"].detach().float().cpu().numpy(),
                                     tn.restore_valid_links(c["links"].detach().float().cpu()).numpy(), ol.numpy(), tl.numpy())
        assert torch.equal(path, torch.from_numpy(ref))
        pick = list(range(0, 64, 16))     # and the torch restatement itself on a few
        assert torch.equal(path[pick], _torch_path(c["match"].detach().cpu()[pick], c["links"].detach().cpu()[pick], ol[pick], tl[pick]))
        for b in range(c["B"]):
            nodes = path_nodes(path[b])
            assert len(nodes) == int(tl[b]) and nodes[0] == 0 and nodes[-1] == int(ol[b]) - 1


def test_long_graph_uses_workspace_trace():
    """Configuration 4 at full size (B=16, L<=1024, T<=256, pre-training scale), every sample."""
    c = workloads.dag_config(4, device=DEV)
    assert c["B"] == 16
    with torch.no_grad():
        path = dagx.dag_best_alignment(c["match"], c["links"], c["out_len"], c["tgt_len"]).cpu()
    ref, _ = cref.best_alignment(c["match"].cpu().numpy(), tn.restore_valid_links(c["links"].cpu()).numpy(),
                                 c["out_len"].cpu().numpy(), c["tgt_len"].cpu().numpy())
    assert torch.equal(path, torch.from_numpy(ref))
    assert torch.equal(path[:2], _torch_path(c["match"].cpu()[:2], c["links"].cpu()[:2], c["out_len"].cpu()[:2], c["tgt_len"].cpu()[:2]))
    m = c["match"].requires_grad_(); lk = c["links"].requires_grad_()
    loss = dagx.dag_loss(m, lk, c["out_len"], c["tgt_len"])
    (loss * c["grad_out"]).sum().backward()
    rloss, rgm, rgl = oracle_loss_and_grads(c["match"].detach().cpu(), c["links"].detach().cpu(),
                                            c["out_len"].cpu(), c["tgt_len"].cpu(), c["grad_out"].cpu())
    assert_close(loss.detach().cpu(), rloss, 1e-4, "loss")
    # block offsets are float64 and residuals float32, so 1e-4 holds even though |alpha| ~ 3.6e3 here
    assert_close(m.grad.cpu(), rgm, 1e-4, "grad_match")
    assert_close(lk.grad.cpu(), rgl, 1e-4, "grad_links")


def test_log_domain_kernels_agree_with_tile_kernels():
    """The one-workgroup log-domain kernels (fallback for flagged samples and L > 1024) must give
    the same loss, gradients and path as the tile-resident kernels; both are checked against the oracle."""
    from da_transformer_amd import _native as nat
    B, L, T = 5, 200, 21
    match, links_sq, ol, tl = random_problem(31, B, L, T, dtype=torch.float32, drop=0.05)
    links = tn.extract_valid_links(links_sq)
    g = torch.randn(B, generator=torch.Generator().manual_seed(2))
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    rpath = _torch_path(match, links, ol, tl)
    results = []
    for on in (1, 0):
        before = nat.lib().dagx_force_log_domain(on)
        try:
            loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
            path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
        finally:
            nat.lib().dagx_force_log_domain(before)
        assert_close(loss, rloss, 1e-4, f"loss (log_domain={on})")
        assert_close(gm, rgm, 1e-4, f"grad_match (log_domain={on})")
        assert_close(gl, rgl, 1e-4, f"grad_links (log_domain={on})")
        feasible = torch.isfinite(rloss)
        assert torch.equal(path[feasible], rpath[feasible])
        results.append((loss, path))
    assert torch.equal(results[0][1], results[1][1])


@pytest.mark.parametrize("shape", [(5, 200, 21, torch.float32), (3, 700, 130, torch.float16)])
def test_alignment_of_samples_the_pipeline_gave_up_on(shape):
    """dagx_best_alignment does a sample that its tile pipeline gave up on again, inside the backtrack launch, by the
    one-workgroup method.  The test switch marks every sample that way (the pipeline itself still runs), with the
    back-pointers in LDS (first shape) and in the workspace (second shape: T*L too large for LDS)."""
    from da_transformer_amd import _native as nat
    B, L, T, dt = shape
    match, links_sq, ol, tl = random_problem(57, B, L, T, dtype=torch.float32)
    match = match.to(dt); links = tn.extract_valid_links(links_sq).to(dt)
    rpath = _torch_path(match, links, ol, tl)
    paths = []
    for mode in (2, 0):
        before = nat.lib().dagx_force_log_domain(mode)
        try:
            paths.append(dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu())
        finally:
            nat.lib().dagx_force_log_domain(before)
    assert torch.equal(paths[0], paths[1])
    assert torch.equal(paths[0], rpath)


def test_alignment_calls_in_a_row_and_on_a_second_stream():
    """Calls of different shapes in a row on one stream (each clears its pipeline words itself, whatever the last call
    left in the reused workspace), then the same on a second stream and again on the first: all must give the
    reference path."""
    problems = []
    for seed, (B, L, T) in enumerate([(8, 200, 31), (3, 520, 40), (11, 130, 17), (8, 200, 31)]):
        match, links_sq, ol, tl = random_problem(300 + seed, B, L, T, dtype=torch.float32)
        links = tn.extract_valid_links(links_sq)
        problems.append((match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV), _torch_path(match, links, ol, tl)))
    other = torch.cuda.Stream(device=DEV)
    for stream in (torch.cuda.current_stream(DEV), other, torch.cuda.current_stream(DEV)):
        stream.wait_stream(torch.cuda.current_stream(DEV))
        with torch.cuda.stream(stream):
            paths = [dagx.dag_best_alignment(m, lk, ol, tl) for m, lk, ol, tl, _ in problems]
        stream.synchronize()
        for path, (_, _, _, _, ref) in zip(paths, problems):
            assert torch.equal(path.cpu(), ref)


@pytest.mark.parametrize("need_grad", [False, True])
@pytest.mark.parametrize("where", [[(1, 3, 2), (2, 150, 40)], [(0, 0, 0), (3, 100, 5)], [(2, 60, 130), (1, 197, 1)]])
def test_nan_transition_gives_what_the_reference_gives(where, need_grad):
    """A NaN among the transitions: the sample's loss is NaN exactly where the torch-native recurrence's is (a NaN on
    some path, also one whose other terms at that cell are all -inf), and finite and equal elsewhere (a NaN outside
    the graph, or in another sample).  With gradients asked for, the loss is the beta sweep's read-out."""
    B, L, T = 4, 200, 21
    match, links_sq, ol, tl = random_problem(5, B, L, T, dtype=torch.float32)
    links = tn.extract_valid_links(links_sq)
    for b, i, d in where:
        links[b, i, d] = float("nan")
    ref = tn.torch_dag_loss(match, tn.restore_valid_links(links), ol, tl)
    loss = dagx.dag_loss(match.to(DEV).requires_grad_(need_grad), links.to(DEV), ol.to(DEV), tl.to(DEV)).detach().cpu()
    assert torch.equal(torch.isnan(loss), torch.isnan(ref)) and torch.isnan(ref).any()
    ok = ~torch.isnan(ref)
    assert_close(loss[ok], ref[ok], 1e-4, "loss of the samples without a NaN")


def test_graph_beyond_tile_limit():
    """L = 1100 > 1024: only the log-domain kernels apply."""
    B, L, T = 2, 1100, 12
    match, links_sq, ol, tl = random_problem(41, B, L, T, dtype=torch.float32)
    links = tn.extract_valid_links(links_sq)
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)
    assert_close(loss, rloss, 1e-4, "loss")
    assert_close(gm, rgm, 1e-4, "grad_match")
    assert_close(gl, rgl, 1e-4, "grad_links")
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert torch.equal(path, _torch_path(match, links, ol, tl))


def test_empty_and_minimal_shapes():
    # empty batch
    m = torch.zeros(0, 3, 4, device=DEV); lk = torch.zeros(0, 4, 3, device=DEV)
    ol = torch.zeros(0, dtype=torch.long, device=DEV); tl = torch.zeros(0, dtype=torch.long, device=DEV)
    assert dagx.dag_loss(m, lk, ol, tl).shape == (0,)
    assert dagx.dag_best_alignment(m, lk, ol, tl).shape == (0, 4)
    # single target / single node, and the smallest real graph
    match = torch.tensor([[[-1.5, -9.0]], [[-0.25, -7.0]]])          # [2, T=1, L=2]
    links = torch.tensor([[[-0.5], [NEG_INF]], [[-0.5], [NEG_INF]]])  # [2, L=2, translen=1]
    ol = torch.tensor([1, 2]); tl = torch.tensor([1, 1])
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert loss[0].item() == pytest.approx(-1.5) and loss[1].item() == -math.inf   # T_b=1 needs L_b=1
    assert gm[0, 0, 0].item() == pytest.approx(1.0) and (gm[1] == 0).all() and (gl == 0).all()
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert path.tolist() == [[0, -1], [-1, -1]]
    match = torch.tensor([[[-1.0, -5.0], [-6.0, -2.0]]])              # T=2, L=2: the single path 0 -> 1
    loss, gm, gl = hip_loss_and_grads(match, links[:1], torch.tensor([2]), torch.tensor([2]))
    assert loss[0].item() == pytest.approx(-3.5)
    assert gm[0].tolist() == [[pytest.approx(1.0), 0.0], [0.0, pytest.approx(1.0)]] and gl[0, 0, 0].item() == pytest.approx(1.0)


def test_alignment_unreachable_end_and_bf16():
    """translen too short to reach the last node -> all -1; bf16 inputs stay bit-exact (exact upcast)."""
    B, L, T = 3, 130, 9
    match, links_sq, ol, tl = random_problem(51, B, L, T, dtype=torch.float32, ragged=False)
    links = tn.extract_valid_links(links_sq, 8)            # (T-1)*8+1 = 65 < 130
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert (path == -1).all()
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert (loss == -math.inf).all() and (gm == 0).all() and (gl == 0).all()
    mb = match.to(torch.bfloat16); lb = tn.extract_valid_links(links_sq).to(torch.bfloat16)
    path = dagx.dag_best_alignment(mb.to(DEV), lb.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert torch.equal(path, _torch_path(mb, lb, ol, tl))


def test_input_checks():
    m = torch.zeros(2, 3, 4, device=DEV); lk = torch.zeros(2, 4, 3, device=DEV)
    ol = torch.tensor([4, 4], device=DEV); tl = torch.tensor([3, 3], device=DEV)
    with pytest.raises(RuntimeError):
        dagx.dag_loss(m, lk[:1], ol, tl)
    with pytest.raises(RuntimeError):
        dagx.dag_loss(m, lk, ol.int(), tl)
    with pytest.raises(RuntimeError):
        dagx.dag_loss(m.to(torch.int32), lk, ol, tl)
    with pytest.raises(RuntimeError):
        dagx.dag_best_alignment(m, torch.zeros(2, 5, 3, device=DEV), ol, tl)


def _peaked_case(seed, B, L, T, link_scale, logit_std, dtype):
    c = workloads.peaked_config(seed, B, L, T, link_scale, logit_std, dtype=dtype)
    match, links, ol, tl = c["match"], c["links"], c["out_len"], c["tgt_len"]
    g = c["grad_out"] * (1024.0 if dtype != torch.float32 else 1.0)     # keep 16-bit gradients out of the subnormals
    return match, links, ol, tl, g


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("L,T,B", [(150, 40, 8), (512, 64, 16), (1024, 256, 4)])
@pytest.mark.parametrize("link_scale,logit_std", [(10.0, 5.0), (30.0, 10.0)])
def test_peaked_inputs_every_sample_against_the_oracle(L, T, B, link_scale, logit_std, dtype):
    """Inputs like a trained model's (most transitions tens to hundreds of nats under the best one, wrong tokens
    at -30 ... -100, pinned nodes): every sample against the float64 oracle, with the default routing (tile
    kernels, whatever they hand to the log-domain kernels) and with the log-domain kernels alone."""
    from da_transformer_amd import _native as nat
    from da_transformer_amd.custom_ops.dag_loss import DagLossFunc
    match, links, ol, tl, g = _peaked_case(1000 + L + int(link_scale), B, L, T, link_scale, logit_std, dtype)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    assert torch.isfinite(rloss).all()
    rtol = RTOL[dtype]
    for on in (0, 1):
        before = nat.lib().dagx_force_log_domain(on)
        try:
            loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
            wide = int((DagLossFunc.last_sample_flags == 2).sum().item())
            redone = int((DagLossFunc.last_sample_flags == 1).sum().item())
        finally:
            nat.lib().dagx_force_log_domain(before)
        print(f"peaked L={L} T={T} links x{link_scale} {dtype}: log_domain={on}: of {B} samples, {wide} settled by the "
              f"float64 tile sweeps, {redone} by the log-domain kernel")
        assert_close(loss, rloss, 1e-4, f"loss (log_domain={on})")
        assert_close(gm.float(), rgm, rtol, f"grad_match (log_domain={on})")
        assert_close(gl.float(), rgl, rtol, f"grad_links (log_domain={on})")


@pytest.mark.parametrize("with_grad", [True, False])
@pytest.mark.parametrize("L,T,B,translen,dtype", [(512, 64, 8, 100, torch.float32), (512, 64, 8, 200, torch.float16),
                                                  (700, 90, 6, 150, torch.float32), (960, 120, 4, 300, torch.bfloat16)])
def test_float64_tile_sweeps_with_limited_transitions(L, T, B, translen, dtype, with_grad):
    """Sharply peaked inputs whose transitions reach translen < L - 1 nodes ahead: the float64 tile sweeps then sum
    over a window of predecessor blocks (not over every lower block), in graphs of 8 to 15 blocks split over 2 to 10
    workgroups.  Most samples must be settled by them, and every sample must match the float64 oracle."""
    from da_transformer_amd.custom_ops.dag_loss import DagLossFunc
    c = workloads.peaked_config(4000 + L + translen, B, L, T, 30.0, 10.0, dtype=dtype, translen=translen)
    match, links, ol, tl = c["match"], c["links"], c["out_len"], c["tgt_len"]
    g = c["grad_out"] * (1024.0 if dtype != torch.float32 else 1.0)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    assert torch.isfinite(rloss).all()
    if with_grad:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    else:
        with torch.no_grad():
            loss = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    flags = DagLossFunc.last_sample_flags.cpu()
    wide, redone = int((flags == 2).sum()), int((flags == 1).sum())
    print(f"peaked x30 L={L} T={T} translen={translen} {dtype}: of {B} samples, {wide} settled by the float64 tile sweeps, "
          f"{redone} by the log-domain kernel")
    assert wide >= B // 2, flags.tolist()
    assert_close(loss, rloss, 1e-4, "loss")
    if with_grad:
        assert_close(gm.float(), rgm, RTOL[dtype], "grad_match")
        assert_close(gl.float(), rgl, RTOL[dtype], "grad_links")


@pytest.mark.parametrize("translen", [5, 32, 100])
def test_log_domain_kernels_with_limited_transitions(translen):
    """translen < L - 1 through the log-domain sweeps and the one-workgroup alignment (every sample forced there):
    the lanes that share a node's transitions must stop at the node's translen-th neighbour."""
    from da_transformer_amd import _native as nat
    B, L, T = 5, 300, 70
    match, links_sq, ol, tl = random_problem(88, B, L, T, dtype=torch.float32, translen=translen)
    ol = torch.minimum(ol, (tl - 1) * translen + 1)           # keep a path possible
    ol[0], tl[0] = min(L, (T - 1) * translen + 1), T
    links = tn.extract_valid_links(links_sq, translen)
    g = torch.randn(B, generator=torch.Generator().manual_seed(3))
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    rpath = _torch_path(match, links, ol, tl)
    before = nat.lib().dagx_force_log_domain(1)
    try:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
        with torch.no_grad():
            alpha_loss = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
        path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    finally:
        nat.lib().dagx_force_log_domain(before)
    assert_close(loss, rloss, 1e-4, "loss (beta read-out)")
    assert_close(alpha_loss, rloss, 1e-4, "loss (alpha read-out)")
    assert_close(gm, rgm, 1e-4, "grad_match")
    assert_close(gl, rgl, 1e-4, "grad_links")
    feasible = torch.isfinite(rloss)
    assert feasible.any() and torch.equal(path[feasible], rpath[feasible])


@pytest.mark.parametrize("log_domain", [0, 1])
def test_long_targets_with_gradients(log_domain):
    """T = 400 > 300 with L = 512: loss and both gradients through the tile kernels and through the
    log-domain kernels (whose gradient kernel walks the steps in chunks, so T is not limited by LDS)."""
    from da_transformer_amd import _native as nat
    B, L, T = 2, 512, 400
    match, links_sq, ol, tl = random_problem(61, B, L, T, dtype=torch.float32)
    ol[0], tl[0] = L, T
    links = tn.extract_valid_links(links_sq)
    g = torch.tensor([1.0, -0.5])
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    before = nat.lib().dagx_force_log_domain(log_domain)
    try:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    finally:
        nat.lib().dagx_force_log_domain(before)
    assert_close(loss, rloss, 1e-4, "loss")
    assert_close(gm, rgm, 1e-4, "grad_match")
    assert_close(gl, rgl, 1e-4, "grad_links")


def test_documented_size_limits_launch():
    """L = 8192 (the largest supported graph: the log-domain kernel's LDS request exceeds the default 64 KiB cap)."""
    B, L, T = 1, 8192, 3
    ol = torch.tensor([L]); tl = torch.tensor([T])
    match = torch.full((B, T, L), -1.0)
    links = torch.full((B, L, 8), -2.0)            # translen 8: reaching node 8191 in 2 steps is impossible
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert loss[0] == -math.inf and (gm == 0).all() and (gl == 0).all()
    # a feasible one of the same size: three targets over nodes 0 -> 8183 -> 8191 needs translen >= 8183
    links = torch.full((B, L, L - 1), NEG_INF); links[0, 0, 8182] = -0.5; links[0, 8183, 7] = -0.25
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert loss[0].item() == pytest.approx(-3.75)
    assert gl[0, 0, 8182].item() == pytest.approx(1.0) and gl[0, 8183, 7].item() == pytest.approx(1.0)
    assert gl.sum().item() == pytest.approx(2.0)


@pytest.mark.parametrize("seed", [0, 1])
def test_reference_self_check_workload(seed):
    """The workload of the reference's own self-check (fs_plugins/custom_ops/dag_loss.py:384-398, 528-533):
    tarlen in [40, 60], bsz = 4096 // tarlen, prelen = 8 * tarlen, translen = 32, match ~ U(0,1), links =
    log_softmax(U(0,1)) over the 32 transitions (finite entries past the last node included, which the
    operators must ignore), lengths shortened by 0..4 -- with its tolerances (loss rtol 1e-3 / atol 1e-4 there;
    1e-4 here) against the float64 oracle."""
    import random
    random.seed(seed)
    gen = torch.Generator().manual_seed(seed)
    tarlen = random.randint(40, 60)
    bsz, prelen, translen = 4096 // tarlen, 8 * tarlen, 32
    match = torch.rand(bsz, tarlen, prelen, generator=gen)
    links = torch.rand(bsz, prelen, translen, generator=gen).log_softmax(-1)
    ol = prelen - torch.randint(0, 5, (bsz,), generator=gen)
    tl = tarlen - torch.randint(0, 5, (bsz,), generator=gen)
    g = torch.full((bsz,), 1.0 / bsz)
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    # the oracle's square layout has no place for transitions that leave the sample: cut them as the operators do
    sq = tn.restore_valid_links(links.double())
    sq = sq.masked_fill(torch.arange(prelen).view(1, 1, -1) >= ol.view(-1, 1, 1), NEG_INF)
    rloss, rgm, rgl_sq = cref.dag_loss_grad(match.double().numpy(), sq.numpy(), ol.numpy(), tl.numpy(), g.double().numpy())
    rgl = tn.extract_valid_links(torch.from_numpy(rgl_sq), translen)
    rgl = rgl.masked_fill(torch.isinf(rgl), 0.0)
    assert torch.isfinite(torch.from_numpy(rloss)).all()
    assert_close(loss, torch.from_numpy(rloss), 1e-4, "loss")
    assert_close(gm, torch.from_numpy(rgm), 1e-4, "grad_match")
    assert_close(gl, rgl, 1e-4, "grad_links")
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    ref, _ = cref.best_alignment(match.numpy(), sq.float().numpy(), ol.numpy(), tl.numpy())
    assert torch.equal(path, torch.from_numpy(ref))


def test_float64_inputs():
    """The reference dispatches double as well (dag_loss.cu:160, dag_best_alignment.cu:150,
    logsoftmax_gather.cu:46-58): float64 tensors run through float64 kernels, and the results and gradients come
    back as float64 to float64 accuracy (tests/test_gpu_float64.py has the wider cases)."""
    B, L, T, V = 3, 70, 11, 257
    match, links_sq, ol, tl = random_problem(71, B, L, T, dtype=torch.float64)
    links = tn.extract_valid_links(links_sq)
    g = torch.tensor([0.5, -1.0, 2.0], dtype=torch.float64)
    m = match.to(DEV).requires_grad_(); lk = links.to(DEV).requires_grad_()
    loss = dagx.dag_loss(m, lk, ol.to(DEV), tl.to(DEV))
    assert loss.dtype == torch.float64
    loss.masked_fill_(loss.isinf(), 0)                       # the criterion's in-place fill works on it
    (loss * g.to(DEV)).sum().backward()
    assert m.grad.dtype == torch.float64 and lk.grad.dtype == torch.float64
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    assert_close(loss.detach().cpu(), rloss, 1e-10, "loss")
    assert_close(m.grad.cpu(), rgm, 1e-10, "grad_match")
    assert_close(lk.grad.cpu(), rgl, 1e-10, "grad_links")
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert torch.equal(path, tn.torch_dag_best_alignment(match, links_sq, ol, tl))
    # gather
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(B, L, V, generator=gen, dtype=torch.float64)
    idx = torch.randint(0, V, (B, T), generator=gen).unsqueeze(1).expand(-1, L, -1)
    xg = x.to(DEV).requires_grad_()
    work = xg * 1
    out, sel = dagx.dag_logsoftmax_gather_inplace(work, idx.to(DEV))
    assert sel.dtype == torch.float64 and out is work
    w = torch.randn(B, L, T, generator=gen, dtype=torch.float64)
    (sel * w.to(DEV)).sum().backward()
    xr = x.clone().requires_grad_()
    rsel = torch.log_softmax(xr, -1).gather(-1, idx)
    (rsel * w).sum().backward()
    assert torch.allclose(sel.detach().cpu(), rsel.detach(), rtol=1e-12, atol=1e-12)
    assert torch.allclose(xg.grad.cpu(), xr.grad, rtol=1e-12, atol=1e-12 * xr.grad.abs().max().item())


@pytest.mark.parametrize("scale,std", [(1.0, 1.0), (10.0, 5.0), (30.0, 10.0)])
def test_no_grad_forward_runs_the_alpha_sweep_alone(scale, std):
    """Without gradients the forward is the alpha sweep only (the reference's choice, dag_loss.cu:346-371); its
    read-out must equal the oracle on benign and on peaked inputs (the latter through the log-domain kernel where
    transitions are too small for the tile arithmetic)."""
    c = workloads.peaked_config(77, 12, 512, 64, scale, std)
    rloss, _, _ = oracle_loss_and_grads(c["match"], c["links"], c["out_len"], c["tgt_len"])
    with torch.no_grad():
        loss = dagx.dag_loss(c["match"].to(DEV), c["links"].to(DEV), c["out_len"].to(DEV), c["tgt_len"].to(DEV))
    assert_close(loss.cpu(), rloss, 1e-4, "loss (alpha read-out)")


def test_calls_on_two_streams_keep_their_own_pipeline_words():
    """The forward's pipeline words are kept per (device, stream): calls enqueued on two streams, which may run
    at the same time, give what the same calls give one after the other."""
    c = workloads.dag_config(1, device=DEV, B=16, dtype=torch.float32)
    c2 = workloads.peaked_config(3, 16, 512, 64, 10.0, 5.0, device=DEV)
    jobs = [(c["match"], c["links"], c["out_len"], c["tgt_len"]), (c2["match"], c2["links"], c2["out_len"], c2["tgt_len"])]

    def run(job):
        m = job[0].detach().requires_grad_(); lk = job[1].detach().requires_grad_()
        loss = dagx.dag_loss(m, lk, job[2], job[3])
        loss.masked_fill(~torch.isfinite(loss), 0).sum().backward()
        return loss.detach(), m.grad, lk.grad

    ref = [run(j) for j in jobs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [None, None]
    for rep in range(3):
        for k, st in enumerate(streams):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                got[k] = run(jobs[k])
        torch.cuda.synchronize()
        for k in range(2):
            for a, b, what in zip(got[k], ref[k], ("loss", "grad_match", "grad_links")):
                assert torch.equal(a, b), f"stream {k}, repetition {rep}: {what} differs from the sequential result"


def test_a_refused_call_leaves_later_calls_intact():
    """An argument error (raised before anything is launched) must not disturb the calls after it."""
    match, links_sq, ol, tl = random_problem(5, 4, 70, 9, dtype=torch.float32, ragged=True)
    links = tn.extract_valid_links(links_sq)
    before = hip_loss_and_grads(match, links, ol, tl)
    with pytest.raises(RuntimeError):
        dagx.dag_loss(match.to(DEV), links.to(DEV)[:, :-1], ol.to(DEV), tl.to(DEV))   # graph sizes disagree
    after = hip_loss_and_grads(match, links, ol, tl)
    for a, b in zip(before, after):
        assert torch.equal(a, b)
