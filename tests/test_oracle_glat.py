"""Pins the oracle's restatement of the glancing glue (oracle.torch_native.glat_glance / glat_mix,
following fs_plugins/criterions/nat_dag_loss.py:273-311) without the reference: a case worked by
hand, the two limits of the keep probability, and plain Python loops on random cases."""
import numpy as np
import torch

from oracle import torch_native as tn


def random_case(seed, B=5, L=23, T=9, vocab=30, pinned=True):
    g = torch.Generator().manual_seed(seed)
    tgt_len = torch.randint(2, T + 1, (B,), generator=g)
    path = torch.full((B, L), -1, dtype=torch.long)
    for b in range(B):
        nodes = torch.randperm(L, generator=g)[: int(tgt_len[b])].sort().values
        path[b, nodes] = torch.arange(int(tgt_len[b]))
    tgt = torch.randint(4, vocab, (B, T), generator=g)
    pred = torch.randint(4, vocab, (B, L), generator=g)
    # make a good share of the predictions right
    right = torch.rand(B, L, generator=g) < 0.4
    pred = torch.where(right & (path >= 0), tgt.gather(1, path.clip(min=0)), pred)
    prev = torch.randint(4, vocab, (B, L), generator=g)
    mask = (torch.rand(B, L, generator=g) < 0.2) & (path >= 0) if pinned else torch.zeros(B, L, dtype=torch.bool)
    rand = torch.rand(B, L, generator=g)
    return path, tgt, pred, prev, mask, tgt_len, rand


def test_glance_case_worked_by_hand():
    # one sample, 6 nodes, 3 targets (tokens 7 8 9); the path emits them at nodes 0, 2, 5
    path = torch.tensor([[0, -1, 1, -1, -1, 2]])
    tgt = torch.tensor([[7, 8, 9]])
    pred = torch.tensor([[7, 7, 5, 8, 9, 9]])          # right at nodes 0 and 5; node 1's 7 equals
    prev = torch.tensor([[2, 3, 3, 3, 3, 3]])          # tgt[0] but node 1 is unassigned
    mask = torch.tensor([[False, False, False, False, False, True]])   # node 5 already pinned
    tgt_len = torch.tensor([3])
    rand = torch.tensor([[0.10, 0.0, 0.20, 0.0, 0.0, 0.99]])
    oracle, same, kp, keep, tokens, force = tn.glat_glance(path, tgt, pred, prev, mask, tgt_len, 0.5, rand)
    assert oracle.tolist() == [[7, 7, 8, 7, 7, 9]]
    assert same.tolist() == [1]                        # node 0 only: node 5 is pinned, node 1 unassigned
    # (3 targets - 1 pinned - 1 right) / 3 * 0.5 = 1/6 on assigned nodes
    want = np.float32(np.float32(1.0) / np.float32(3.0)) * np.float32(0.5)
    assert kp.tolist() == [[want, 0.0, want, 0.0, 0.0, want]]
    assert keep.tolist() == [[True, False, False, False, False, True]]   # 0.10 < 1/6 <= 0.20; node 5 pinned
    assert tokens.tolist() == [[7, 3, 3, 3, 3, 9]]
    assert force.tolist() == [[0, -1, -1, -1, -1, 2]]


def test_keep_probability_limits():
    path, tgt, pred, prev, mask, tgt_len, rand = random_case(3)
    # context_p = 0: only the already pinned nodes stay revealed
    out = tn.glat_glance(path, tgt, pred, prev, mask, tgt_len, 0.0, rand)
    assert torch.equal(out[3], mask)
    assert torch.equal(out[5], path.masked_fill(~mask, -1))
    # nothing predicted right, nothing pinned, context_p = 1, rand = 0: every assigned node is revealed
    wrong = torch.zeros_like(pred)
    none = torch.zeros_like(mask)
    out = tn.glat_glance(path, tgt, wrong, prev, none, tgt_len, 1.0, torch.zeros_like(rand))
    assert out[1].tolist() == [0] * path.shape[0]
    assert torch.equal(out[3], path >= 0)
    assert torch.equal(out[4], torch.where(path >= 0, tgt.gather(1, path.clip(min=0)), prev))
    assert torch.equal(out[5], path)


def test_glance_equals_python_loops():
    for seed in range(4):
        path, tgt, pred, prev, mask, tgt_len, rand = random_case(10 + seed, pinned=seed % 2 == 0)
        p = 0.37
        oracle, same, kp, keep, tokens, force = tn.glat_glance(path, tgt, pred, prev, mask, tgt_len, p, rand)
        B, L = path.shape
        for b in range(B):
            same_b = sum(1 for j in range(L) if path[b, j] >= 0 and not mask[b, j] and pred[b, j] == tgt[b, path[b, j]])
            assert int(same[b]) == same_b
            prob = np.float32(np.float32(int(tgt_len[b]) - int(mask[b].sum()) - same_b) / np.float32(int(tgt_len[b]))) * np.float32(p)
            for j in range(L):
                a = int(path[b, j])
                assert int(oracle[b, j]) == int(tgt[b, max(a, 0)])
                assert float(kp[b, j]) == (float(prob) if a >= 0 else 0.0)
                k = bool(mask[b, j]) or float(rand[b, j]) < float(kp[b, j])
                assert bool(keep[b, j]) == k
                assert int(tokens[b, j]) == (int(oracle[b, j]) if k else int(prev[b, j]))
                assert int(force[b, j]) == (a if k else -1)


def test_oracle_reproduces_the_glancing_fixture():
    import os
    from conftest import ROOT
    z = np.load(os.path.join(ROOT, "tests", "golden", "glance_small.npz"))
    t = {k: torch.from_numpy(z[k]) for k in z.files if z[k].ndim > 0}
    out = tn.glat_glance(t["path"], t["tgt_tokens"], t["pred_tokens"], t["prev_output_tokens"], t["prev_mask"], t["tgt_len"],
                         float(z["context_p"]), t["rand"])
    for got, key in zip(out, ("oracle", "same_num", "keep_prob", "keep_word_mask", "glat_prev_output_tokens", "next_force_emit")):
        assert torch.equal(got, t[key]), key
    assert torch.equal(tn.force_alignment(t["match"], t["next_force_emit"]), t["forced_match"])
