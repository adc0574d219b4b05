"""GPU parity of the criterion glue (dag_force_alignment, dag_glat_glance / _oracle / _mix, through
the C ABI) against the CPU oracle.  Integer, byte and mask outputs are compared bit for bit, and
so are the rewritten match tensor and the keep probability."""
import pytest
import torch

import da_transformer_amd as dagx
from oracle import torch_native as tn
from helpers import random_problem
from test_oracle_glat import random_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _same(got, want):
    """Bit-level equality that also accepts NaN == NaN and tells -0.0 from +0.0."""
    got = got.cpu()
    assert got.dtype == want.dtype and got.shape == want.shape
    if got.dtype.is_floating_point:
        as_int = {4: torch.int32, 2: torch.int16}[got.element_size()]
        assert torch.equal(got.contiguous().view(as_int), want.contiguous().view(as_int))
    else:
        assert torch.equal(got, want)


def _force_case(seed, B, T, L, dup=False):
    gen = torch.Generator().manual_seed(seed)
    force = torch.full((B, L), -1, dtype=torch.long)
    for b in range(B):
        n = int(torch.randint(0, min(T, L) + 1, (1,), generator=gen)) if b else 0      # sample 0: nothing forced
        nodes = torch.randperm(L, generator=gen)[:n].sort().values
        force[b, nodes] = torch.randperm(T, generator=gen)[:n].sort().values
    if dup and B > 1 and L > 3:
        force[1, 1] = 0; force[1, 3] = 0                                               # two nodes name target 0
    return force


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,T,L", [(3, 7, 20), (4, 16, 64), (2, 9, 300), (1, 1, 1)])
@pytest.mark.parametrize("transposed", [False, True])
def test_force_alignment_forward_is_bit_exact(dtype, B, T, L, transposed):
    gen = torch.Generator().manual_seed(B * 100 + T)
    match = torch.randn(B, T, L, generator=gen).to(dtype)
    match[0, 0, 0] = -0.0                        # passes through an addition of +0.0 in the reference
    if L > 2:
        match[-1, -1, 2] = float("-inf")
    force = _force_case(T + L, B, T, L, dup=True)
    want = tn.force_alignment(match, force)
    dev = match.to(DEV)
    if transposed:                               # the criterion's view: [B,L,T] storage, transposed
        dev = dev.transpose(1, 2).contiguous().transpose(1, 2)
    got = dagx.dag_force_alignment(dev, force.to(DEV))
    assert got.is_contiguous()
    _same(got, want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_force_alignment_gradient(dtype):
    B, T, L = 4, 11, 37
    gen = torch.Generator().manual_seed(5)
    match = torch.randn(B, T, L, generator=gen).to(dtype)
    force = _force_case(9, B, T, L, dup=True)
    grad = torch.randn(B, T, L, generator=gen).to(dtype)
    m = match.clone().requires_grad_()
    tn.force_alignment(m, force).backward(grad)
    d = match.to(DEV).requires_grad_()
    dagx.dag_force_alignment(d, force.to(DEV)).backward(grad.to(DEV).transpose(1, 2).contiguous().transpose(1, 2))
    _same(d.grad, m.grad)


def test_forced_loss_and_gradients_through_dag_loss():
    """force -> dag_loss, the order of NATDAGLoss._compute_dag_loss (nat_dag_loss.py:178-188)."""
    B, T, L = 4, 9, 40
    match, links, ol, tl = random_problem(77, B, L, T, dtype=torch.float32)
    # pin, in every sample, the node that a feasible path can give to target 3
    force = torch.full((B, L), -1, dtype=torch.long)
    force[:, 10] = 3
    m = match.clone().requires_grad_(); s = links.clone().requires_grad_()
    want = tn.torch_dag_loss(tn.force_alignment(m, force), s, ol, tl)
    g = -1.0 / (B * tl.float())
    want.backward(g)
    dm = match.to(DEV).requires_grad_(); ds = tn.extract_valid_links(links).to(DEV).requires_grad_()
    got = dagx.dag_loss(dagx.dag_force_alignment(dm, force.to(DEV)), ds, ol.to(DEV), tl.to(DEV))
    got.backward(g.to(DEV))
    assert torch.isfinite(want).all()
    assert torch.allclose(got.cpu(), want.detach(), rtol=1e-4)                    # fp32: rtol 1e-4
    gl = tn.extract_valid_links(s.grad)
    gl = gl.masked_fill(gl == float("-inf"), 0.0)                                 # the converter pads with -inf
    for a, b in ((dm.grad.cpu(), m.grad), (ds.grad.cpu(), gl)):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-4 * float(b.abs().max()))
    assert (dm.grad[:, 3] == 0).all()


@pytest.mark.parametrize("B,L,T", [(5, 23, 9), (3, 300, 40), (64, 512, 64), (2, 1000, 3)])
@pytest.mark.parametrize("pinned", [True, False, None])
def test_glat_glance_is_bit_exact(B, L, T, pinned):
    path, tgt, pred, prev, mask, tgt_len, rand = random_case(B + L, B=B, L=L, T=T, vocab=50, pinned=bool(pinned))
    p = 0.43
    want = tn.glat_glance(path, tgt, pred, prev, mask, tgt_len, p, rand)
    dmask = None if pinned is None else mask.to(DEV)
    got = dagx.dag_glat_glance(path.to(DEV), tgt.to(DEV), pred.to(DEV), prev.to(DEV), tgt_len.to(DEV), p,
                               glat_prev_mask=dmask, rand=rand.to(DEV))
    assert got.keep_word_mask.dtype == torch.bool
    for g, w in zip(got, want):
        _same(g, w)
    # the two-stage route of the strategies that compute their own keep probability
    oracle, same = dagx.dag_glat_oracle(path.to(DEV), tgt.to(DEV), pred.to(DEV), dmask)
    _same(oracle, want[0]); _same(same, want[1])
    keep_prob = torch.rand(B, L, generator=torch.Generator().manual_seed(1))
    w3 = tn.glat_mix(path, want[0], prev, keep_prob, rand, mask)
    g3 = dagx.dag_glat_mix(path.to(DEV), oracle, prev.to(DEV), keep_prob.to(DEV), rand.to(DEV), dmask)
    for g, w in zip(g3, w3):
        _same(g, w)


def test_glat_glance_after_the_alignment_kernel():
    """dag_best_alignment -> dag_glat_glance -> dag_force_alignment, the second pass's inputs."""
    B, T, L = 6, 12, 50
    match, links, ol, tl = random_problem(21, B, L, T, dtype=torch.float32)
    gen = torch.Generator().manual_seed(2)
    tgt = torch.randint(4, 60, (B, T), generator=gen); pred = torch.randint(4, 60, (B, L), generator=gen)
    prev = torch.full((B, L), 3); rand = torch.rand(B, L, generator=gen)
    path = dagx.dag_best_alignment(match.to(DEV), tn.extract_valid_links(links).to(DEV), ol.to(DEV), tl.to(DEV))
    assert torch.equal(path.cpu(), tn.torch_dag_best_alignment(match, links, ol, tl))
    got = dagx.dag_glat_glance(path, tgt.to(DEV), pred.to(DEV), prev.to(DEV), tl.to(DEV), 0.5, rand=rand.to(DEV))
    want = tn.glat_glance(path.cpu(), tgt, pred, prev, torch.zeros(B, L, dtype=torch.bool), tl, 0.5, rand)
    for g, w in zip(got, want):
        _same(g, w)
    forced = dagx.dag_force_alignment(match.to(DEV), got.next_force_emit)
    _same(forced, tn.force_alignment(match, want[5]))


def test_glue_argument_errors():
    z = torch.zeros(2, 3, 4, device=DEV)
    with pytest.raises(RuntimeError):
        dagx.dag_force_alignment(z, torch.zeros(2, 5, dtype=torch.long, device=DEV))
    with pytest.raises(RuntimeError):
        dagx.dag_force_alignment(z, torch.zeros(2, 4, dtype=torch.int32, device=DEV))
    with pytest.raises(RuntimeError):
        dagx.dag_force_alignment(z.cpu(), torch.zeros(2, 4, dtype=torch.long))
    path = torch.zeros(2, 4, dtype=torch.long, device=DEV)
    with pytest.raises(RuntimeError):
        dagx.dag_glat_glance(path, path, path.int(), path, torch.ones(2, dtype=torch.long, device=DEV), 0.5)
    with pytest.raises(RuntimeError):
        dagx.dag_glat_mix(path, path, path, torch.zeros(2, 4, device=DEV), torch.zeros(2, 5, device=DEV))


def test_glancing_golden_fixture():
    import os
    import numpy as np
    from conftest import ROOT
    z = np.load(os.path.join(ROOT, "tests", "golden", "glance_small.npz"))
    t = {k: torch.from_numpy(z[k]) for k in z.files if z[k].ndim > 0}
    d = {k: v.to(DEV) for k, v in t.items()}
    got = dagx.dag_glat_glance(d["path"], d["tgt_tokens"], d["pred_tokens"], d["prev_output_tokens"], d["tgt_len"],
                               float(z["context_p"]), glat_prev_mask=d["prev_mask"], rand=d["rand"])
    for g, key in zip(got, ("oracle", "same_num", "keep_prob", "keep_word_mask", "glat_prev_output_tokens", "next_force_emit")):
        _same(g, t[key])
    _same(dagx.dag_force_alignment(d["match"], got.next_force_emit), t["forced_match"])
