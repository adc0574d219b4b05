"""The float64 operators (float64 arithmetic throughout, kernels of their own) against the float64 oracles, to
float64 tolerances: 1e-10 where the float32 operators are held to 1e-4.  The reference instantiates its kernels for
double as well (fs_plugins/custom_ops/dag_loss.cu:160, dag_best_alignment.cu:150, logsoftmax_gather.cu:343-347)."""
import pytest
import torch

import da_transformer_amd as dagx
from oracle import cref
from oracle import torch_native as tn
from helpers import random_problem, NEG_INF
from test_gpu_dag import hip_loss_and_grads, oracle_loss_and_grads, assert_close
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-10


@pytest.mark.parametrize("B,L,T,translen,drop", [
    (3, 70, 11, None, 0.0), (6, 150, 40, 32, 0.0), (5, 150, 40, 5, 0.0), (4, 300, 64, None, 0.5),
    (2, 1030, 30, 200, 0.0), (8, 512, 64, None, 0.0), (1, 9, 9, None, 0.0), (2, 40, 2, None, 0.0)])
def test_loss_and_gradients(B, L, T, translen, drop):
    match, links_sq, ol, tl = random_problem(100 + L, B, L, T, translen=translen, drop=drop)
    if B >= 4:
        ol[1], tl[1] = L, T
        ol[2], tl[2] = max(2, L // 3), 2
        ol[3], tl[3] = max(T, L // 2), T          # (little slack)
    links = tn.extract_valid_links(links_sq, translen)
    g = torch.randn(B, generator=torch.Generator().manual_seed(1), dtype=torch.float64)
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    assert loss.dtype == torch.float64 and gm.dtype == torch.float64 and gl.dtype == torch.float64
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    assert_close(loss, rloss, TOL, "loss")
    assert_close(gm, rgm, TOL, "grad_match")
    assert_close(gl, rgl, TOL, "grad_links")
    with torch.no_grad():
        loss0 = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert torch.equal(loss0, loss), "the forward without gradients is the same alpha sweep"


def test_sharply_peaked_inputs_and_levels_far_apart():
    """What takes the float32 operators three kernels is one code path here: transitions of -300 nats and match
    values a thousand nats apart lie within float64 log-domain sums."""
    c = workloads.peaked_config(5, 6, 512, 64, 30.0, 10.0)
    match, links, ol, tl, g = c["match"].double(), c["links"].double(), c["out_len"], c["tgt_len"], c["grad_out"].double().cpu()
    match = match + torch.where(torch.rand(match.shape, generator=torch.Generator().manual_seed(2)) < 0.3, -1000.0, 0.0)
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl, g)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl, g)
    assert_close(loss, rloss, TOL, "loss")
    assert_close(gm, rgm, 1e-9, "grad_match")
    assert_close(gl, rgl, 1e-9, "grad_links")


def test_samples_without_a_path_and_invalid_lengths():
    B, L, T = 5, 60, 12
    match, links_sq, ol, tl = random_problem(9, B, L, T)
    links_sq[1, 0, :] = NEG_INF                    # node 0 has no successor: no path
    ol[2], tl[2] = 5, 9                            # T_b > L_b
    ol[3], tl[3] = L + 3, T                        # L_b beyond the tensor
    match[4, 3, :] = NEG_INF                       # a target nobody can emit
    links = tn.extract_valid_links(links_sq)
    loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    assert torch.isfinite(loss[0]) and (loss[1:] == NEG_INF).all()
    assert (gm[1:] == 0).all() and (gl[1:] == 0).all() and torch.isfinite(gm).all() and torch.isfinite(gl).all()
    rloss, rgm, rgl = oracle_loss_and_grads(match[:1], links[:1], ol[:1], tl[:1])
    assert_close(loss[:1], rloss, TOL, "loss"); assert_close(gm[:1], rgm, TOL, "grad_match"); assert_close(gl[:1], rgl, TOL, "grad_links")
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert (path[1:] == -1).all() and (path[0] >= 0).sum() == tl[0]


def test_gradcheck_through_the_public_operator():
    """Only an operator that really computes in float64 passes torch's finite-difference check at its default
    tolerances."""
    B, L, T = 2, 9, 4
    match, links_sq, ol, tl = random_problem(3, B, L, T)
    links = tn.extract_valid_links(links_sq)
    links = links.masked_fill(torch.isinf(links), -40.0)     # finite everywhere, so that every entry can be perturbed
    m = match.to(DEV).requires_grad_(); lk = links.to(DEV).requires_grad_()
    assert torch.autograd.gradcheck(lambda a, b: dagx.dag_loss(a, b, ol.to(DEV), tl.to(DEV)), (m, lk), eps=1e-6, atol=1e-7, rtol=1e-5)


def test_strided_match_and_mixed_dtypes():
    B, L, T = 4, 130, 20
    match, links_sq, ol, tl = random_problem(17, B, L, T)
    links = tn.extract_valid_links(links_sq)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)
    stored = match.transpose(1, 2).contiguous().to(DEV).requires_grad_()       # [B,L,T] storage, read as [B,T,L]
    lk = links.to(DEV).requires_grad_()
    loss = dagx.dag_loss(stored.transpose(1, 2), lk, ol.to(DEV), tl.to(DEV))
    loss.sum().backward()
    assert_close(loss.detach().cpu(), rloss, TOL, "loss")
    assert_close(stored.grad.transpose(1, 2).cpu(), rgm, TOL, "grad_match")
    assert_close(lk.grad.cpu(), rgl, TOL, "grad_links")
    # float64 match with float32 links: the links are cast up, their gradient comes back as float32
    lk32 = links.float().to(DEV).requires_grad_()
    m = match.to(DEV).requires_grad_()
    loss = dagx.dag_loss(m, lk32, ol.to(DEV), tl.to(DEV))
    assert loss.dtype == torch.float64
    loss.sum().backward()
    assert lk32.grad.dtype == torch.float32 and m.grad.dtype == torch.float64
    r2, rgm2, rgl2 = oracle_loss_and_grads(match, links.float().double(), ol, tl)
    assert_close(loss.detach().cpu(), r2, TOL, "loss"); assert_close(m.grad.cpu(), rgm2, TOL, "grad_match")
    assert_close(lk32.grad.cpu(), rgl2, 1e-6, "grad_links (rounded to float32)")


def _torch_path64(match, links, ol, tl):
    sq = tn.restore_valid_links(links)
    return tn.torch_dag_best_alignment(match, sq, ol, tl)


@pytest.mark.parametrize("B,L,T,translen", [(6, 150, 40, None), (4, 300, 30, 17), (3, 1030, 25, None), (8, 512, 64, None)])
def test_best_alignment_against_the_torch_native_rule_in_float64(B, L, T, translen):
    match, links_sq, ol, tl = random_problem(200 + L, B, L, T, translen=translen)
    links = tn.extract_valid_links(links_sq, translen)
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV))
    assert path.dtype == torch.int64
    ref = _torch_path64(match, links, ol, tl)
    # (a sample without any path, which a short translen can make, gets -1 everywhere; the torch-native rule walks
    #  back through -inf scores there)
    feasible = torch.isfinite(tn.torch_dag_max_score(match, tn.restore_valid_links(links), ol, tl))
    assert torch.equal(path.cpu()[feasible], ref[feasible]) and (path.cpu()[~feasible] == -1).all()


def test_best_alignment_ties_and_differences_below_float32():
    """Quantised scores (many exact ties: the lowest predecessor must win) and two paths whose scores differ in the
    twelfth digit (float32 scores would tie them and take the lower index, float64 must take the better)."""
    B, L, T = 4, 90, 14
    gen = torch.Generator().manual_seed(5)
    match = torch.randint(-3, 1, (B, T, L), generator=gen).double()
    sq = torch.randint(-2, 1, (B, L, L), generator=gen).double()
    sq = sq.masked_fill(torch.triu(torch.ones(L, L), 1) == 0, NEG_INF)
    ol = torch.tensor([L, L - 1, L - 7, L]); tl = torch.tensor([T, T - 1, T, 2])
    links = tn.extract_valid_links(sq)
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert torch.equal(path, _torch_path64(match, links, ol, tl))
    # 0 -> 1 -> 3 and 0 -> 2 -> 3, the second better by 1e-12
    match = torch.zeros(1, 3, 4, dtype=torch.float64)
    sq = torch.full((1, 4, 4), NEG_INF, dtype=torch.float64)
    sq[0, 0, 1] = -1.0; sq[0, 0, 2] = -1.0 + 1e-12; sq[0, 1, 3] = -1.0; sq[0, 2, 3] = -1.0
    ol = torch.tensor([4]); tl = torch.tensor([3])
    links = tn.extract_valid_links(sq)
    path = dagx.dag_best_alignment(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert path.tolist() == [[0, -1, 1, 2]]
    assert dagx.dag_best_alignment(match.float().to(DEV), links.float().to(DEV), ol.to(DEV), tl.to(DEV)).cpu().tolist() == [[0, 1, -1, 2]]


@pytest.mark.parametrize("V,S,transposed", [(257, 11, False), (1000, 64, True), (37, 300, False), (40000, 5, False)])
def test_logsoftmax_gather(V, S, transposed):
    B, L = 3, 20
    gen = torch.Generator().manual_seed(V)
    x = torch.randn(B, L, V, generator=gen, dtype=torch.float64) * 5
    idx = torch.randint(0, V, (B, L, S), generator=gen)
    idx[0, 0, :] = idx[0, 0, 0]                       # one row gathers the same id S times
    if S >= 11:
        idx[1, 3, 4:9] = idx[1, 3, 2]
    w = torch.randn(B, L, S, generator=gen, dtype=torch.float64)
    xg = x.to(DEV).requires_grad_()
    work = xg * 1
    out, sel = dagx.dag_logsoftmax_gather_inplace(work, idx.to(DEV), transposed)
    assert sel.dtype == torch.float64 and out is work and sel.shape == (B, L, S)
    if transposed:
        assert sel.transpose(1, 2).is_contiguous()
    assert torch.equal(work.detach().cpu(), x), "the forward only reads the logits"
    (sel * w.to(DEV)).sum().backward()
    want, lse = cref.lsg(x.view(-1, V).numpy(), idx.view(-1, S).numpy())
    assert_close(sel.detach().cpu().reshape(-1, S), torch.from_numpy(want), 1e-12, "selected")
    ref = cref.lsg_bwd(x.view(-1, V).numpy(), idx.view(-1, S).numpy(), w.view(-1, S).numpy())
    assert_close(xg.grad.cpu().view(-1, V), torch.from_numpy(ref), 1e-12, "gradient of the logits")
    # ids outside the vocabulary give NaN instead of a fault, and no gradient
    bad = idx.clone(); bad[2, 5, 0] = V; bad[2, 6, 0] = -1
    with torch.no_grad():
        _, sel2 = dagx.dag_logsoftmax_gather_inplace(x.to(DEV), bad.to(DEV))
    assert torch.isnan(sel2[2, 5, 0]) and torch.isnan(sel2[2, 6, 0]) and torch.isnan(sel2).sum() == 2
