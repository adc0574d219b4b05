"""The replay harness itself (tests/criterion_replay.py), without a GPU: the oracle's torch restatement and the
plain-C restatement, driven through the same call sequence, must agree on every stage."""
import torch

import criterion_replay as cr


def test_two_oracle_operator_sets_agree_through_the_replay():
    B, L, T, V = 3, 40, 9, 300
    ol = torch.tensor([40, 31, 22]); tl = torch.tensor([9, 5, 8])
    inp = cr.make_step_inputs(7, B, L, T, V, ol, tl)
    a = cr.criterion_like(cr.torch_oracle_ops(), context_p=0.5, **inp)
    b = cr.criterion_like(cr.c_oracle_ops(), context_p=0.5, **inp)
    assert a["logits_unchanged_by_no_grad_gather"] and b["logits_unchanged_by_no_grad_gather"]
    assert torch.equal(a["path"], b["path"]) and torch.equal(a["force_emit"], b["force_emit"])
    assert (a["force_emit"] >= 0).any() and int(a["invalid_nsentences"]) == 0
    for k in ("loss", "per_sample", "grad_logits", "grad_links"):
        ref = b[k].double()
        assert torch.allclose(a[k].double(), ref, rtol=1e-4, atol=1e-4 * ref.abs().max().item()), k
    # every path visits exactly T_b nodes, from node 0 to node L_b - 1
    for r in range(B):
        nodes = [j for j, t in enumerate(a["path"][r].tolist()) if t >= 0]
        assert len(nodes) == int(tl[r]) and nodes[0] == 0 and nodes[-1] == int(ol[r]) - 1


def test_replay_without_glancing_and_with_an_infeasible_sample():
    B, L, T, V = 2, 20, 6, 50
    ol = torch.tensor([20, 4]); tl = torch.tensor([6, 6])          # sample 1: T_b > L_b
    inp = cr.make_step_inputs(9, B, L, T, V, ol, tl)
    a = cr.criterion_like(cr.torch_oracle_ops(), context_p=0.5, glat=False, **inp)
    b = cr.criterion_like(cr.c_oracle_ops(), context_p=0.5, glat=False, **inp)
    assert int(a["invalid_nsentences"]) == 1 == int(b["invalid_nsentences"])
    assert a["per_sample"][1] == 0 and torch.allclose(a["per_sample"], b["per_sample"], rtol=1e-5)
    # the reference's torch form still sends a gradient to match[T_b-1, L_b-1] of an infeasible sample
    # (the `+ match` behind a fully masked logsumexp), the kernels' convention is zero: compare sample 0 only
    assert torch.allclose(a["grad_links"][0], b["grad_links"][0], rtol=1e-4, atol=1e-9)
    assert torch.allclose(a["grad_logits"][0], b["grad_logits"][0], rtol=1e-4, atol=1e-9)
