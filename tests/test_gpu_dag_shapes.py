"""Many small shapes drawn at random (seeded): graph sizes around the block edges of the tile kernels, short and long
targets, limited transitions, dropped transitions, batch sizes that are no multiple of eight, wide dynamic ranges --
each through the default routing (float32 tile sweeps, then float64, then log domain) and with the float64 sweeps
first, with gradients and without, against the float64 oracle."""
import pytest
import torch

import da_transformer_amd as dagx
from da_transformer_amd.custom_ops.dag_loss import DagLossFunc
from oracle import torch_native as tn
from helpers import random_problem
from test_gpu_dag import hip_loss_and_grads, oracle_loss_and_grads, assert_close, _torch_path

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _draw(seed):
    gen = torch.Generator().manual_seed(1000 + seed)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=gen))
    L = [r(2, 70), r(60, 70), r(120, 200), r(250, 330), r(380, 520), r(630, 710), r(900, 1024)][seed % 7]
    T = max(2, min(L, [r(2, 4), r(2, 40), r(20, 90), r(2, 12)][(seed // 7) % 4]))
    B = [1, 3, 5, 9, 12][(seed // 3) % 5]
    translen = [None, None, r(1, 6), r(20, 70), r(100, 300)][(seed // 2) % 5]
    if translen is not None:
        translen = min(translen, L - 1) if L > 1 else None
        if translen is not None and translen < 1:
            translen = None
    scale = [1.0, 1.0, 8.0, 40.0][(seed // 5) % 4]       # match values N(0,1) * scale - 2
    drop = [0.0, 0.3, 0.0][(seed // 11) % 3]
    return B, L, T, translen, scale, drop


@pytest.mark.parametrize("float64_first", [False, True])
@pytest.mark.parametrize("seed", range(42))
def test_random_shapes(seed, float64_first):
    B, L, T, translen, scale, drop = _draw(seed)
    match, links_sq, ol, tl = random_problem(seed, B, L, T, dtype=torch.float32, drop=drop, translen=translen, match_scale=scale)
    if translen is not None:      # keep a path possible for most samples: T_b - 1 steps of at most translen nodes
        ol = torch.minimum(ol, (tl - 1) * translen + 1).clamp_(min=1)
        tl = torch.minimum(tl, ol)
    links = tn.extract_valid_links(links_sq, translen)
    g = torch.randn(B, generator=torch.Generator().manual_seed(seed))
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    before = dagx.dag_loss_float64_first(float64_first)
    try:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
        flags = DagLossFunc.last_sample_flags.cpu().tolist()
        with torch.no_grad():
            loss0 = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    finally:
        dagx.dag_loss_float64_first(before)
    what = f"B={B} L={L} T={T} translen={translen} scale={scale} drop={drop} flags={flags}"
    if float64_first:
        assert all(f in (1, 2) for f in flags), what
    assert_close(loss, rloss, 1e-4, "loss: " + what)
    assert_close(loss0, rloss, 1e-4, "loss without gradients: " + what)
    assert_close(gm, rgm, 1e-4, "grad_match: " + what)
    assert_close(gl, rgl, 1e-4, "grad_links: " + what)
    if not float64_first:
        feasible = torch.isfinite(rloss)
        path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
        rpath = _torch_path(match, links, ol, tl)
        assert torch.equal(path[feasible], rpath[feasible]), "alignment: " + what
