"""Pins for the best-alignment, log-softmax-gather and layout oracles; CPU only."""
import math

import numpy as np
import pytest
import torch

from oracle import brute, cref
from oracle import torch_native as tn
from helpers import random_problem, path_nodes, NEG_INF


def _rescore(match, links, nodes):
    s = sum(match[t, j] for t, j in enumerate(nodes))
    return s + sum(links[a, b] for a, b in zip(nodes[:-1], nodes[1:]))


@pytest.mark.parametrize("seed", range(8))
def test_alignment_equals_brute_force_argmax(seed):
    B, L, T = 3, 8, 4
    match, links, out_len, tgt_len = random_problem(300 + seed, B, L, T, dtype=torch.float32,
                                                    drop=0.2 if seed % 2 else 0.0)
    path = tn.torch_dag_best_alignment(match, links, out_len, tgt_len)
    cpath, cscore = cref.best_alignment(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    score = tn.torch_dag_max_score(match, links, out_len, tgt_len)
    assert path.shape == (B, L) and path.dtype == torch.int64
    for b in range(B):
        best, arg = brute.best_path(match[b].double().tolist(), links[b].double().tolist(),
                                    int(out_len[b]), int(tgt_len[b]))
        if not arg:   # the random edge drop left no path: only the convention is checked
            assert (cpath[b] == -1).all() and cscore[b] == -math.inf
            continue
        assert len(arg) == 1, "random continuous inputs should be tie-free"
        assert path_nodes(path[b]) == list(arg[0])
        assert path_nodes(torch.from_numpy(cpath[b])) == list(arg[0])
        assert score[b].item() == pytest.approx(best, rel=1e-5)
        assert cscore[b] == score[b].item()      # same fp32 roundings


def test_alignment_tie_rule_all_equal_scores():
    """All finite links 0 and match 0: every path ties; lowest-index backtrack gives
    nodes 0,1,...,T_b-2,L_b-1."""
    B, L, T = 3, 12, 6
    out_len = torch.tensor([12, 9, 7]); tgt_len = torch.tensor([6, 4, 2])
    match = torch.zeros(B, T, L)
    i = torch.arange(L).view(1, L, 1); j = torch.arange(L).view(1, 1, L)
    links = torch.zeros(B, L, L).masked_fill(~((j > i) & (j < out_len.view(B, 1, 1))), NEG_INF)
    path = tn.torch_dag_best_alignment(match, links, out_len, tgt_len)
    cpath, _ = cref.best_alignment(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    for b in range(B):
        want = list(range(int(tgt_len[b]) - 1)) + [int(out_len[b]) - 1]
        assert path_nodes(path[b]) == want
        assert path_nodes(torch.from_numpy(cpath[b])) == want


@pytest.mark.parametrize("seed", range(6))
def test_alignment_with_quantised_values_matches_c_restatement(seed):
    """Coarsely quantised inputs make exact ties frequent; the torch restatement (library
    max, first index) and the C restatement (explicit lowest index) must agree bit for bit."""
    B, L, T = 4, 40, 11
    match, links, out_len, tgt_len = random_problem(400 + seed, B, L, T, dtype=torch.float32)
    match = (match * 2).round() / 2
    links = ((links * 2).round() / 2).masked_fill(torch.isinf(links), NEG_INF)
    path = tn.torch_dag_best_alignment(match, links, out_len, tgt_len)
    cpath, cscore = cref.best_alignment(match.numpy(), links.numpy(), out_len.numpy(), tgt_len.numpy())
    assert np.array_equal(path.numpy(), cpath)
    score = tn.torch_dag_max_score(match, links, out_len, tgt_len)
    for b in range(B):
        nodes = path_nodes(path[b])
        Lb, Tb = int(out_len[b]), int(tgt_len[b])
        assert len(nodes) == Tb and nodes[0] == 0 and nodes[-1] == Lb - 1
        assert all(a < c for a, c in zip(nodes[:-1], nodes[1:]))
        assert _rescore(match[b], links[b], nodes).item() == pytest.approx(score[b].item(), rel=1e-6)
        assert sorted(t for t in path[b].tolist() if t >= 0) == list(range(Tb))


def test_logsoftmax_gather_oracles():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(2, 5, 37, generator=g, dtype=torch.float64)
    idx = torch.randint(0, 37, (2, 5, 6), generator=g)
    idx[0, 0, 1] = idx[0, 0, 0]           # a duplicated id
    same, sel = tn.torch_dag_logsoftmax_gather_inplace(x.float(), idx)
    assert same.dtype == torch.float32 and sel.dtype == torch.float32 and sel.shape == (2, 5, 6)
    csel, clse = cref.lsg(x.view(10, 37).numpy(), idx.view(10, 6).numpy())
    assert np.allclose(csel, sel.view(10, 6).numpy(), rtol=1e-5, atol=1e-6)
    assert np.allclose(clse, torch.logsumexp(x.view(10, 37), -1).numpy(), rtol=1e-13)
    # backward: autograd through the torch oracle == explicit softmax-Jacobian form in C
    xr = x.clone().requires_grad_()
    _, sel64 = tn.torch_dag_logsoftmax_gather_inplace(xr, idx)
    # (dtype=float32 inside the oracle; compare at fp32 accuracy)
    gout = torch.randn(2, 5, 6, generator=g, dtype=torch.float32)
    gx = torch.autograd.grad((sel64 * gout).sum(), xr)[0]
    cgx = cref.lsg_bwd(x.view(10, 37).numpy(), idx.view(10, 6).numpy(), gout.view(10, 6).double().numpy())
    assert np.allclose(cgx, gx.view(10, 37).numpy(), rtol=1e-5, atol=1e-6)
    # each row of the gradient sums to zero (softmax Jacobian annihilates constants)
    assert np.allclose(cgx.sum(-1), 0, atol=1e-12)


def test_layout_round_trip():
    _, links, out_len, _ = random_problem(2, 3, 9, 4)
    for translen in (None, 8, 3, 1):
        sh = tn.extract_valid_links(links, translen)
        tl = 8 if translen is None else translen
        assert sh.shape == (3, 9, tl)
        back = tn.restore_valid_links(sh)
        i = torch.arange(9).view(1, 9, 1); j = torch.arange(9).view(1, 1, 9)
        band = (j > i) & (j - i <= tl)
        assert torch.equal(back[band.expand(3, -1, -1)], links[band.expand(3, -1, -1)])
        assert torch.isinf(back[~band.expand(3, -1, -1)]).all()
        # shifted entry [i, d] is square entry [i, i+d+1]
        for ii in range(9):
            for d in range(tl):
                jj = ii + d + 1
                if jj < 9:
                    assert torch.equal(sh[:, ii, d], links[:, ii, jj])
                else:
                    assert torch.isinf(sh[:, ii, d]).all()


def test_force_alignment_fragment_sum_identity():
    """Pinning a node to a target splits the DAG: the forced loss equals the sum of the
    fragment losses with the shared end points counted once (nat_dag_loss.py:122-152)."""
    L, T = 9, 5
    match, links, out_len, tgt_len = random_problem(21, 1, L, T, ragged=False)
    force = torch.full((1, L), -1, dtype=torch.long)
    force[0, 4] = 2                        # node 4 must emit target 2
    fm = tn.force_alignment(match, force)
    assert fm[0, 2, 4] == 0 and torch.isinf(fm[0, 2, :4]).all() and torch.isinf(fm[0, 2, 5:]).all()
    assert torch.equal(fm[0, [0, 1, 3, 4]], match[0, [0, 1, 3, 4]])
    whole = tn.torch_dag_loss(fm, links, out_len, tgt_len)[0]
    left = tn.torch_dag_loss(fm[:, :3, :5], links[:, :5, :5], torch.tensor([5]), torch.tensor([3]))[0]
    right = tn.torch_dag_loss(fm[:, 2:, 4:], links[:, 4:, 4:], torch.tensor([5]), torch.tensor([3]))[0]
    assert whole.item() == pytest.approx((left + right - fm[0, 2, 4]).item(), rel=1e-12)
    # forced rows carry no gradient
    m = match.clone().requires_grad_()
    tn.torch_dag_loss(tn.force_alignment(m, force), links, out_len, tgt_len).sum().backward()
    assert (m.grad[0, 2] == 0).all() and m.grad[0, 1].abs().sum() > 0
