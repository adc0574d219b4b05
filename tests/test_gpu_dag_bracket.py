"""Inputs built so that the path that carries the mass runs through numbers the float32 tile sweeps' linear domain
cannot hold (a cell, a block of cells or a transition more than 126 nats under its scale), next to a weak
alternative the domain holds well.  A sweep that flushes such numbers silently returns the alternative: finite,
wrong, unflagged.  The two sweeps of a sample bracket log Z instead (one rounds every flushed number down, one up),
so each of these samples must be recognised, done again -- by the float64 tile sweeps where they have the range
(sample flag 2), else by the log-domain kernel (flag 1) -- and come out as the float64 oracle has it, with gradients
and under no_grad, in the default routing and with the log-domain kernels alone."""
import math

import pytest
import torch

import da_transformer_amd as dagx
from da_transformer_amd import _native as nat
from da_transformer_amd.custom_ops.dag_loss import DagLossFunc
from oracle import torch_native as tn
from helpers import random_problem, NEG_INF
from test_gpu_dag import hip_loss_and_grads, oracle_loss_and_grads, assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def sparse_case(L, T, cells, edges):
    """One sample: match is -inf but for cells {(t, node): value}, links -inf but for edges {(i, j): value}."""
    match = torch.full((1, T, L), NEG_INF)
    for (t, j), v in cells.items():
        match[0, t, j] = v
    sq = torch.full((1, L, L), NEG_INF)
    for (i, j), v in edges.items():
        sq[0, i, j] = v
    return match, tn.extract_valid_links(sq), torch.tensor([L]), torch.tensor([T])


def cell_under_its_block_maximum():
    """Two cells of one block at step 1, 130 nats apart; the low one carries the only strong continuation
    (log Z = -130.7), the high one a continuation worth -500."""
    h = math.log(0.5)
    return sparse_case(8, 4,
                       {(0, 0): 0.0, (1, 1): -130.0, (1, 2): 0.0, (2, 3): 0.0, (2, 4): -500.0, (3, 7): 0.0},
                       {(0, 1): h, (0, 2): h, (1, 3): 0.0, (2, 4): 0.0, (3, 7): 0.0, (4, 7): 0.0}), -130.0 + h


def cell_flushed_by_both_directions():
    """The same cell is more than 126 nats under a block-mate in the alpha sweep (one with a strong prefix and a
    continuation worth -1000) and under another in the beta sweep (weak prefix, strong continuation): both sweeps
    flush the path that carries the mass (-260) and agree on -1000."""
    t3 = math.log(1.0 / 3.0)
    cells = {(0, 0): 0.0, (4, 10): 0.0,
             (1, 1): -130.0, (2, 4): 0.0, (3, 7): -130.0,       # the path that matters
             (1, 2): 0.0, (2, 5): 0.0, (3, 8): -1000.0,         # strong prefix, hopeless continuation
             (1, 3): -1000.0, (2, 6): 0.0, (3, 9): 0.0}         # hopeless prefix, strong continuation
    edges = {(0, 1): t3, (0, 2): t3, (0, 3): t3, (1, 4): 0.0, (2, 5): 0.0, (3, 6): 0.0,
             (4, 7): 0.0, (5, 8): 0.0, (6, 9): 0.0, (7, 10): 0.0, (8, 10): 0.0, (9, 10): 0.0}
    return sparse_case(11, 5, cells, edges), -260.0 + t3


def block_under_its_neighbour():
    """Predecessor blocks 100 nats apart: the high block reaches the last node through a transition of -120, the
    low block through one of 0 (log Z = -100.7); a scale factor exp(-100) is no float32 number."""
    h = math.log(0.5)
    return sparse_case(192, 3,
                       {(0, 0): 0.0, (1, 1): 0.0, (1, 64): -100.0, (2, 191): 0.0},
                       {(0, 1): h, (0, 64): h, (1, 191): -120.0, (64, 191): 0.0}), -100.0 + h


def transition_under_the_float32_range():
    """The only path crosses a transition of -140: no float32 number in the float32 sweeps' scaling, one in the
    float64 sweeps' (which stage transitions down to -175)."""
    return sparse_case(70, 2, {(0, 0): -1.0, (1, 69): -2.0}, {(0, 69): -140.0}), -143.0


def transition_among_the_subnormals():
    """The only path crosses a transition of -185: scaled like the float64 sweeps' staged transitions it is a subnormal
    float32 number, two bits of fraction at that depth.  Both sweeps of the sample would carry the same wrong value
    (8 % off at -190) and agree on it; such transitions are not staged, and the sample goes to the log-domain kernel."""
    return sparse_case(70, 2, {(0, 0): -1.0, (1, 69): -2.0}, {(0, 69): -185.0}), -188.0


def transition_under_every_range():
    """The only path crosses a transition of -250, which neither tile variant stages."""
    return sparse_case(70, 2, {(0, 0): -1.0, (1, 69): -2.0}, {(0, 69): -250.0}), -253.0


CASES = [cell_under_its_block_maximum, cell_flushed_by_both_directions, block_under_its_neighbour,
         transition_under_the_float32_range, transition_among_the_subnormals, transition_under_every_range]
# which kernel settles the case in the default routing: 2 = the float64 tile sweeps, 1 = the log-domain kernel
ROUTE = {"cell_under_its_block_maximum": 2, "cell_flushed_by_both_directions": 2, "block_under_its_neighbour": 2,
         "transition_under_the_float32_range": 2, "transition_among_the_subnormals": 1, "transition_under_every_range": 1}


@pytest.mark.parametrize("log_domain", [0, 1])
@pytest.mark.parametrize("with_grad", [False, True])
@pytest.mark.parametrize("case", CASES, ids=lambda f: f.__name__)
def test_mass_below_the_linear_domain_is_never_lost_silently(case, with_grad, log_domain):
    (match, links, ol, tl), expected = case()
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)
    assert abs(rloss.item() - expected) < 0.05           # the case is what its description says
    before = nat.lib().dagx_force_log_domain(log_domain)
    try:
        if with_grad:
            loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
        else:
            with torch.no_grad():
                loss = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
        flag = int(DagLossFunc.last_sample_flags.item())
    finally:
        nat.lib().dagx_force_log_domain(before)
    assert flag == (1 if log_domain else ROUTE[case.__name__]), "the float32 sweeps' result must not stand"
    assert_close(loss, rloss, 1e-4, "loss")
    if with_grad:
        assert_close(gm, rgm, 1e-4, "grad_match")
        assert_close(gl, rgl, 1e-4, "grad_links")


@pytest.mark.parametrize("with_grad", [False, True])
def test_cases_in_one_batch_with_benign_samples(with_grad):
    """The crafted samples padded into a batch of ordinary ones: only they are redone."""
    B, L, T = 8, 192, 6
    match, links_sq, ol, tl = random_problem(21, B, L, T, dtype=torch.float32)
    links = tn.extract_valid_links(links_sq)
    hard = []
    for k, case in enumerate(CASES):
        (m, lk, o, t), _ = case()
        b = k + 1
        match[b] = NEG_INF; links[b] = NEG_INF
        match[b, :m.shape[1], :m.shape[2]] = m[0]
        links[b, :lk.shape[1], :lk.shape[2]] = lk[0]
        ol[b], tl[b] = o[0], t[0]
        hard.append(b)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)
    if with_grad:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    else:
        with torch.no_grad():
            loss = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    flags = DagLossFunc.last_sample_flags.cpu().tolist()
    assert flags == [0] + [ROUTE[case.__name__] for case in CASES] + [0] * (B - 1 - len(CASES)), flags
    assert_close(loss, rloss, 1e-4, "loss")
    if with_grad:
        assert_close(gm, rgm, 1e-4, "grad_match")
        assert_close(gl, rgl, 1e-4, "grad_links")


@pytest.mark.parametrize("with_grad", [False, True])
def test_numbers_below_the_range_that_carry_no_mass_cost_nothing(with_grad):
    """Finite transitions of -130 ... -400 and cells hundreds of nats under their block maximum, none of them on
    a path that matters: the sample stays on the tile kernels (no redo) and matches the oracle."""
    B, L, T = 4, 300, 20
    match, links_sq, ol, tl = random_problem(5, B, L, T, dtype=torch.float32, ragged=False)
    gen = torch.Generator().manual_seed(9)
    links = tn.extract_valid_links(links_sq)
    deep = (torch.rand(links.shape, generator=gen) < 0.05) & torch.isfinite(links)
    links = torch.where(deep, links - 130.0 - 270.0 * torch.rand(links.shape, generator=gen), links)
    low = torch.rand(match.shape, generator=gen) < 0.1
    low[:, 0, 0] = False; low[:, -1, -1] = False
    match = torch.where(low, match - 300.0, match)
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)
    if with_grad:
        loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
    else:
        with torch.no_grad():
            loss = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu()
    assert int(DagLossFunc.last_sample_flags.sum().item()) == 0
    assert_close(loss, rloss, 1e-4, "loss")
    if with_grad:
        assert_close(gm, rgm, 1e-4, "grad_match")
        assert_close(gl, rgl, 1e-4, "grad_links")


@pytest.mark.parametrize("with_grad", [False, True])
def test_float64_sweeps_first_gives_the_same_results(with_grad):
    """dag_loss_float64_first(True): no float32 pass; every sample is settled by the float64 tile sweeps (flag 2) or,
    where they cannot (the transition of -250), by the log-domain kernel -- benign and crafted samples alike, equal
    to the oracle; switched off again, benign samples are back on the float32 sweeps."""
    B, L, T = 8, 192, 6
    match, links_sq, ol, tl = random_problem(21, B, L, T, dtype=torch.float32)
    links = tn.extract_valid_links(links_sq)
    for k, case in enumerate(CASES):
        (m, lk, o, t), _ = case()
        b = k + 1
        match[b] = NEG_INF; links[b] = NEG_INF
        match[b, :m.shape[1], :m.shape[2]] = m[0]
        links[b, :lk.shape[1], :lk.shape[2]] = lk[0]
        ol[b], tl[b] = o[0], t[0]
    rloss, rgm, rgl = oracle_loss_and_grads(match, links, ol, tl)

    def run():
        if with_grad:
            loss, gm, gl = hip_loss_and_grads(match, links, ol, tl)
        else:
            with torch.no_grad():
                loss, gm, gl = dagx.dag_loss(match.to(DEV), links.to(DEV), ol.to(DEV), tl.to(DEV)).cpu(), None, None
        return loss, gm, gl, DagLossFunc.last_sample_flags.cpu().tolist()

    before = dagx.dag_loss_float64_first(True)
    try:
        loss, gm, gl, flags = run()
    finally:
        assert dagx.dag_loss_float64_first(before) is True
    assert flags == [2] + [ROUTE[case.__name__] for case in CASES] + [2] * (B - 1 - len(CASES)), flags
    assert_close(loss, rloss, 1e-4, "loss")
    if with_grad:
        assert_close(gm, rgm, 1e-4, "grad_match")
        assert_close(gl, rgl, 1e-4, "grad_links")
    loss, gm, gl, flags = run()
    assert flags == [0] + [ROUTE[case.__name__] for case in CASES] + [0] * (B - 1 - len(CASES)), flags
    assert_close(loss, rloss, 1e-4, "loss (switched off again)")
