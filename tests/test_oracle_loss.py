"""Pins for the DAG-loss oracle (torch restatement + C restatement); CPU only."""
import math

import numpy as np
import pytest
import torch

from oracle import brute, cref
from oracle import torch_native as tn
from helpers import random_problem, NEG_INF


def test_logsumexp_keepdim_matches_library_and_handles_dead_slices():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 5, 7, generator=g, dtype=torch.float64)
    x[0, :, 2] = NEG_INF            # a dead slice along dim 1
    x[1, 3, :] = NEG_INF            # partial -inf
    x.requires_grad_()
    y = tn.logsumexp_keepdim(x, 1)
    ref = torch.logsumexp(x.detach(), 1, keepdim=True)
    assert y.shape == (3, 1, 7)
    assert torch.equal(torch.isinf(y), torch.isinf(ref))
    fin = ~torch.isinf(ref)
    assert torch.allclose(y[fin], ref[fin], rtol=1e-13, atol=0)
    y.masked_fill(torch.isinf(y), 0).sum().backward()
    assert not torch.isnan(x.grad).any()
    assert (x.grad[0, :, 2] == 0).all()
    # live slices: gradient is the softmax
    sm = torch.softmax(x.detach()[2], 0)
    assert torch.allclose(x.grad[2], sm, rtol=1e-12, atol=1e-15)


@pytest.mark.parametrize("seed", range(8))
def test_loss_equals_brute_force_enumeration(seed):
    L, T = 7, 4
    match, links, out_len, tgt_len = random_problem(seed, 3, L, T, drop=0.3 if seed % 2 else 0.0)
    got = tn.torch_dag_loss(match, links, out_len, tgt_len)
    closs, _, _ = cref.dag_loss(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    for b in range(3):
        want = brute.log_likelihood(match[b].tolist(), links[b].tolist(), int(out_len[b]), int(tgt_len[b]))
        if want == -math.inf:
            assert got[b].item() == -math.inf and closs[b] == -math.inf
        else:
            assert got[b].item() == pytest.approx(want, rel=1e-12, abs=1e-12)
            assert closs[b] == pytest.approx(want, rel=1e-12, abs=1e-12)


@pytest.mark.parametrize("seed", range(4))
def test_gradients_equal_brute_force_posteriors(seed):
    L, T = 6, 4
    match, links, out_len, tgt_len = random_problem(100 + seed, 2, L, T, drop=0.25)
    match.requires_grad_(); links.requires_grad_()
    loss = tn.torch_dag_loss(match, links, out_len, tgt_len)
    g = torch.tensor([0.7, -1.3], dtype=torch.float64)
    gm, gl = torch.autograd.grad((loss * g).sum(), [match, links])
    _, cgm, cgl = cref.dag_loss_grad(match.detach().numpy(), links.detach().numpy(),
                                     out_len.numpy(), tgt_len.numpy(), g.numpy())
    for b in range(2):
        node, edge = brute.posteriors(match[b].tolist(), links[b].tolist(), int(out_len[b]), int(tgt_len[b]))
        node = torch.tensor(node, dtype=torch.float64) * g[b]
        edge = torch.tensor(edge, dtype=torch.float64) * g[b]
        assert torch.allclose(gm[b], node, rtol=1e-10, atol=1e-13)
        assert torch.allclose(gl[b], edge, rtol=1e-10, atol=1e-13)
        assert np.allclose(cgm[b], node.numpy(), rtol=1e-10, atol=1e-13)
        assert np.allclose(cgl[b], edge.numpy(), rtol=1e-10, atol=1e-13)


def test_closed_forms_two_targets_and_full_length():
    match, links, _, _ = random_problem(7, 4, 9, 9, ragged=False)
    # T_b = 2: the single path 0 -> L_b-1
    out_len = torch.tensor([9, 8, 5, 2]); tgt_len = torch.tensor([2, 2, 2, 2])
    got = tn.torch_dag_loss(match, links, out_len, tgt_len)
    closs, _, _ = cref.dag_loss(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    for b in range(4):
        last = int(out_len[b]) - 1
        want = match[b, 0, 0] + links[b, 0, last] + match[b, 1, last]
        assert got[b].item() == pytest.approx(want.item(), rel=1e-13)
        assert closs[b] == pytest.approx(want.item(), rel=1e-13)
    # T_b = L_b: the single path 0,1,...,L_b-1
    out_len = torch.tensor([9, 7, 4, 3]); tgt_len = out_len.clone()
    got = tn.torch_dag_loss(match, links, out_len, tgt_len)
    closs, _, _ = cref.dag_loss(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    for b in range(4):
        n = int(out_len[b])
        want = sum(match[b, k, k] for k in range(n)) + sum(links[b, k, k + 1] for k in range(n - 1))
        assert got[b].item() == pytest.approx(want.item(), rel=1e-13)
        assert closs[b] == pytest.approx(want.item(), rel=1e-13)


def test_path_lengths_form_a_distribution():
    """Row-normalised links, match == 0, single sink L_b-1: sum over T_b of exp(loss) == 1."""
    L = 10
    _, links, out_len, _ = random_problem(3, 2, L, L, ragged=False)
    match = torch.zeros(2, L, L, dtype=torch.float64)
    total = torch.zeros(2, dtype=torch.float64)
    for Tb in range(2, L + 1):
        tl = torch.full((2,), Tb)
        total += tn.torch_dag_loss(match, links, out_len, tl).exp()
    assert torch.allclose(total, torch.ones(2, dtype=torch.float64), rtol=1e-12)


@pytest.mark.parametrize("seed", range(3))
def test_posterior_mass_invariants_and_c_restatement(seed):
    B, L, T = 5, 24, 9
    match, links, out_len, tgt_len = random_problem(200 + seed, B, L, T, drop=0.1)
    match.requires_grad_(); links.requires_grad_()
    loss = tn.torch_dag_loss(match, links, out_len, tgt_len)
    g = torch.randn(B, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)
    gm, gl = torch.autograd.grad((loss * g).sum(), [match, links])
    closs, alpha, beta = cref.dag_loss(match.detach().numpy(), links.detach().numpy(),
                                       out_len.numpy(), tgt_len.numpy())
    _, cgm, cgl = cref.dag_loss_grad(match.detach().numpy(), links.detach().numpy(),
                                     out_len.numpy(), tgt_len.numpy(), g.numpy())
    assert np.allclose(closs, loss.detach().numpy(), rtol=1e-12)
    assert np.allclose(cgm, gm.numpy(), rtol=1e-9, atol=1e-14)
    assert np.allclose(cgl, gl.numpy(), rtol=1e-9, atol=1e-14)
    for b in range(B):
        Lb, Tb = int(out_len[b]), int(tgt_len[b])
        assert alpha[b, Tb - 1, Lb - 1] == pytest.approx(beta[b, 0, 0], rel=1e-12)
        # every target position is emitted by exactly one node; T_b-1 edges are used
        assert torch.allclose(gm[b, :Tb].sum(-1), g[b].expand(Tb), rtol=1e-10)
        assert gl[b].sum().item() == pytest.approx(g[b].item() * (Tb - 1), rel=1e-10)
        assert (gm[b, Tb:] == 0).all() and (gm[b, :, Lb:] == 0).all()
        assert (gl[b, Lb:] == 0).all() and (gl[b, :, Lb:] == 0).all()


def test_gradcheck_fp64():
    match, links, out_len, tgt_len = random_problem(5, 2, 6, 4)
    finite = torch.isfinite(links)
    base = links.clone()

    def fn(m, free):
        lk = base.masked_scatter(finite, free)
        return tn.torch_dag_loss(m, lk, out_len, tgt_len)

    free = links[finite].clone().requires_grad_()
    assert torch.autograd.gradcheck(fn, (match.clone().requires_grad_(), free), eps=1e-6, atol=1e-6)


def test_infeasible_sample_gives_minus_inf():
    match, links, out_len, tgt_len = random_problem(9, 2, 6, 4, ragged=False)
    links[0, 0, :] = NEG_INF           # node 0 has no way out
    got = tn.torch_dag_loss(match, links, out_len, tgt_len)
    closs, _, _ = cref.dag_loss(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    assert got[0].item() == -math.inf and closs[0] == -math.inf
    assert math.isfinite(got[1].item())
    _, cgm, cgl = cref.dag_loss_grad(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy(),
                                     np.ones(2))
    assert (cgm[0] == 0).all() and (cgl[0] == 0).all()


def test_fp32_restatement_tracks_fp64():
    match, links, out_len, tgt_len = random_problem(11, 4, 64, 16)
    l64 = tn.torch_dag_loss(match, links, out_len, tgt_len)
    l32 = tn.torch_dag_loss(match.float(), links.float(), out_len, tgt_len)
    assert torch.allclose(l32.double(), l64, rtol=1e-5)
