"""The criterion's call sequence (criterion_replay.py: nat_dag_loss.py:155-203 and :239-321) run with the HIP
operators and with the CPU oracle on the same seeded inputs: configuration 0 and configuration 4 at full size
(B=16, L<=1024, T<=256, V=30522; fp32 and fp16 links)."""
import pytest
import torch

import da_transformer_amd as dagx
import criterion_replay as cr
import workloads
from oracle import torch_native as tn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def close(got, ref, rtol, what):
    got, ref = got.double(), ref.double()
    assert got.shape == ref.shape, what
    assert torch.isfinite(got).all(), what
    atol = rtol * ref.abs().max().item()
    err = (got - ref).abs()
    assert (err <= atol + rtol * ref.abs()).all(), f"{what}: max err {err.max().item():.3e} (atol {atol:.3e})"


def recording(ops, store):
    """ops whose gather also records what it returned (to hand the same `match` to the reference alignment)."""
    def gather(w, idx):
        w, match = ops.gather(w, idx)
        store.append(match)
        return w, match
    return cr.OpSet(gather, ops.loss, ops.align, ops.square_links, ops.device)


def reference_path(match_blt, links_shifted, ol, tl):
    """The torch rule (lowest predecessor among equals) on exactly the match values the HIP gather produced
    (the plain-C restatement, pinned against torch_dag_best_alignment in tests/test_oracle_align_gather.py)."""
    return cr._cref_align(match_blt.transpose(1, 2).float().cpu(), tn.restore_valid_links(links_shifted.float()), ol, tl)


def test_configuration_0_full_replay_both_operator_sets():
    """B=4, L=64, T=16, V=1000 fp32: every stage compared, both sets replayed independently."""
    B, L, T, V = 4, 64, 16, 1000
    ol = torch.tensor([64, 64, 57, 40]); tl = torch.tensor([16, 16, 9, 13])
    inp = cr.make_step_inputs(1234, B, L, T, V, ol, tl)
    for ref_ops in (cr.torch_oracle_ops(), cr.c_oracle_ops()):
        got = cr.criterion_like(cr.hip_ops(DEV), context_p=0.5, **inp)
        ref = cr.criterion_like(ref_ops, context_p=0.5, **inp)
        assert got["logits_unchanged_by_no_grad_gather"]
        assert torch.equal(got["path"], ref["path"]) and torch.equal(got["force_emit"], ref["force_emit"])
        assert torch.equal(got["glat_tokens"], ref["glat_tokens"])
        assert int(got["invalid_nsentences"]) == 0 == int(ref["invalid_nsentences"])
        close(got["per_sample"], ref["per_sample"], 1e-4, "per-sample loss")
        close(got["loss"], ref["loss"], 1e-4, "loss")
        close(got["grad_logits"], ref["grad_logits"], 1e-4, "grad logits")
        close(got["grad_links"], ref["grad_links"], 1e-4, "grad links")


def test_in_place_fill_of_the_returned_loss_with_and_without_grad():
    """nat_dag_loss.py:190-191 verbatim on the operator's output; an infeasible sample is zeroed, its
    gradients are zero, and the same lines work under no_grad (validation)."""
    from helpers import random_problem
    B, L, T = 5, 40, 8
    match, links_sq, _, _ = random_problem(17, B, L, T, dtype=torch.float32, ragged=False)
    ol = torch.tensor([40, 40, 5, 40, 33], device=DEV); tl = torch.tensor([8, 8, 8, 2, 6], device=DEV)   # sample 2: T_b > L_b
    match = match.to(DEV)
    links = workloads.make_links_shifted(torch.Generator().manual_seed(5), ol.cpu(), L, "cpu").to(DEV)
    m = match.detach().requires_grad_(); lk = links.detach().requires_grad_()
    loss_result = dagx.dag_loss(m, lk, ol, tl)
    invalid_masks = loss_result.isinf().logical_or(loss_result.isnan())
    loss_result.masked_fill_(invalid_masks, 0)
    assert invalid_masks.tolist() == [False, False, True, False, False] and loss_result[2] == 0
    (-(loss_result / tl).mean()).backward()
    assert (m.grad[2] == 0).all() and (lk.grad[2] == 0).all() and torch.isfinite(m.grad).all()
    g = (-1.0 / (B * tl.double())).float().cpu()
    from test_gpu_dag import oracle_loss_and_grads, assert_close
    keep = [0, 1, 3, 4]
    rloss, rgm, rgl = oracle_loss_and_grads(match.cpu()[keep], links.cpu()[keep], ol.cpu()[keep], tl.cpu()[keep], g[keep])
    assert_close(loss_result.detach().cpu()[keep], rloss, 1e-4, "loss")
    assert_close(m.grad.cpu()[keep], rgm, 1e-4, "grad_match")
    assert_close(lk.grad.cpu()[keep], rgl, 1e-4, "grad_links")
    with torch.no_grad():
        l2 = dagx.dag_loss(match, links, ol, tl)
        l2.masked_fill_(l2.isinf().logical_or(l2.isnan()), 0)
    assert_close(l2.cpu()[keep], rloss, 1e-4, "loss under no_grad (alpha read-out)")
    # gradients of one input only
    for which in (0, 1):
        m = match.detach().requires_grad_(which == 0); lk = links.detach().requires_grad_(which == 1)
        out = dagx.dag_loss(m, lk, ol, tl)
        out.masked_fill_(out.isinf(), 0)
        (-(out / tl).mean()).backward()
        if which == 0:
            assert lk.grad is None
            assert_close(m.grad.cpu()[keep], rgm, 1e-4, "grad_match alone")
        else:
            assert m.grad is None
            assert_close(lk.grad.cpu()[keep], rgl, 1e-4, "grad_links alone")


@pytest.mark.parametrize("links_dtype", [torch.float32, torch.float16])
def test_configuration_4_full_size(links_dtype):
    """B=16, L<=1024, T<=256, V=30522, fp16 logits: gather -> best alignment -> glancing -> gather (grad) ->
    force-emit -> dag_loss -> in-place fill -> backward to logits and links, as one chain."""
    c = workloads.dag_config(4, device="cpu", B=1)     # only for the shape constants
    B, L, T, V = 16, c["L"], c["T"], c["V"]
    gen = torch.Generator().manual_seed(1238)
    ol = 4 * torch.randint(128, 257, (B,), generator=gen); tl = torch.minimum(torch.randint(128, 257, (B,), generator=gen), ol)
    ol[0], tl[0] = L, T
    inp = cr.make_step_inputs(4321, B, L, T, V, ol, tl, logits_dtype=torch.float16, links_dtype=links_dtype)
    recorded = []
    got = cr.criterion_like(recording(cr.hip_ops(DEV), recorded), context_p=0.5, **inp)
    assert got["logits_unchanged_by_no_grad_gather"]
    assert int(got["invalid_nsentences"]) == 0
    # alignment: bit-exact with the torch rule on the very match values it was given
    ref_path = reference_path(recorded[0], inp["links"], ol, tl)
    assert torch.equal(got["path"], ref_path)
    kept = (got["force_emit"] >= 0).sum().item()
    assert 0 < kept < (got["path"] >= 0).sum().item()
    # main pass against the float64 C oracle with the same pinned nodes
    ref = cr.criterion_like(cr.c_oracle_ops(), context_p=0.5, glat=False, force_emit=got["force_emit"],
                            **{k: (v.float() if k in ("logits", "links") else v) for k, v in inp.items()})
    rt_links = 1e-4 if links_dtype == torch.float32 else 1e-2
    close(got["per_sample"], ref["per_sample"], 1e-4, "per-sample loss")
    close(got["loss"], ref["loss"], 1e-4, "loss")
    close(got["grad_links"].float(), ref["grad_links"], rt_links, "grad links")
    # fp16 logits: the gradient comes back in fp16 (values ~1e-5: scaled by a loss scale in real training)
    close(got["grad_logits"].float(), ref["grad_logits"], 1e-2, "grad logits")
