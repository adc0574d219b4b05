"""Pins the oracle's restatement of Viterbi decoding (oracle.torch_native.inference_viterbi,
following fs_plugins/models/glat_decomposed_with_link.py:720-777) without the reference: every
path through tiny graphs is enumerated and scored from the definition, and one case is worked
by hand."""
import itertools

import pytest
import torch

from oracle import torch_native as tn
from helpers import random_links_square

NEG_INF = float("-inf")
PAD = 1


def decode_case(seed, B, L, vocab=6, min_len=3):
    gen = torch.Generator().manual_seed(seed)
    out_len = torch.randint(min_len, L + 1, (B,), generator=gen)
    out_len[0] = L
    links = random_links_square(gen, B, L, out_len, dtype=torch.float32, drop=0.2)
    logits = torch.log_softmax(torch.randn(B, L, vocab, generator=gen) * 2, -1)
    u, tok = logits.max(-1)
    return links, u, tok, out_len


def collapse(tokens):
    """The reference's rule read forwards: the last token always stays; an earlier one stays when
    it is not the pad and differs from the token that follows it."""
    n = len(tokens)
    return [t for k, t in enumerate(tokens) if k == n - 1 or (t != PAD and t != tokens[k + 1])]


def best_by_enumeration(links, u, out_len, max_length, beta, joint):
    """arg max over all 0 -> x_0 < ... < x_{n-1} -> L_b-1 in float64, and the runner-up's margin."""
    Lb = int(out_len)
    scored = []
    for n in range(1, max_length + 1):
        for xs in itertools.combinations(range(1, Lb - 1), n):
            chain = (0,) + xs + (Lb - 1,)
            s = sum(float(links[a, b]) for a, b in zip(chain[:-1], chain[1:]))
            s += (float(u[0]) + sum(float(u[x]) for x in xs)) if joint else float(u[xs[0]])
            if s > NEG_INF:
                scored.append((s / n ** beta, xs))
    scored.sort(reverse=True)
    return scored


@pytest.mark.parametrize("joint", [False, True])
@pytest.mark.parametrize("beta", [0.0, 1.0, 0.5])
def test_viterbi_equals_enumeration(joint, beta):
    B, L, scale = 6, 9, 3.0
    links, u, tok, out_len = decode_case(11 + int(joint), B, L)
    max_length = int(2 * L / scale)
    out, pred_len, nodes = tn.inference_viterbi(links, u, tok, out_len, scale, beta, joint, PAD)
    checked = 0
    for b in range(B):
        scored = best_by_enumeration(links[b], u[b], out_len[b], max_length, beta, joint)
        if not scored:
            continue
        if len(scored) > 1 and scored[0][0] - scored[1][0] < 1e-4:
            continue                                     # too close to call in float32
        assert tuple(nodes[b]) == scored[0][1]
        assert int(pred_len[b]) == len(scored[0][1])
        want = collapse([int(tok[b, x]) for x in scored[0][1]])
        got = [t for t in out[b].tolist()]
        assert got[:len(want)] == want and all(t == PAD for t in got[len(want):])
        checked += 1
    assert checked >= 4


def test_viterbi_case_worked_by_hand():
    # 5 nodes; transitions (probabilities): 0->1 .5, 0->2 .5, 1->2 .5, 1->4 .5, 2->3 .5, 2->4 .5, 3->4 1
    p = torch.zeros(1, 5, 5)
    p[0, 0, 1] = .5; p[0, 0, 2] = .5; p[0, 1, 2] = .5; p[0, 1, 4] = .5; p[0, 2, 3] = .5; p[0, 2, 4] = .5; p[0, 3, 4] = 1.
    links = p.log()
    u = torch.tensor([[0.9, 0.5, 0.8, 0.8, 0.9]]).log()
    tok = torch.tensor([[0, 7, 8, 8, 2]])
    out_len = torch.tensor([5])
    # joint, no length penalty (beta 0): 0-1-4: .9*.5*.5*.5 = .1125; 0-2-4: .9*.5*.8*.5 = .18;
    # 0-1-2-4: .9*.5*.5*.5*.8*.5 = .045; 0-2-3-4: .9*.5*.8*.5*.8*1 = .144 -> 0-2-4 wins, one token
    out, n, nodes = tn.inference_viterbi(links, u, tok, out_len, 2.5, 0.0, True, PAD)
    assert nodes == [[2]] and n.tolist() == [1] and out.tolist() == [[8]]
    # beta 1 divides the log score by the length: log(.18)/1 = -1.71 against log(.144)/2 = -0.97 and
    # log(.0288)/3 = -1.18 (0-1-2-3-4) -> 0-2-3-4 wins; its tokens 8 8 collapse to one
    out, n, nodes = tn.inference_viterbi(links, u, tok, out_len, 2.5, 1.0, True, PAD)
    assert nodes == [[2, 3]] and n.tolist() == [2] and out.tolist() == [[8]]
    # plain form: only the first interior node's token counts: 0-1-...: .5*.5(u1) ; 0-2-3-4: .5*.8*.5*1 = .2;
    # 0-2-4: .5*.8*.5 = .2 as well -> with beta 0 the shorter length comes first in the arg max over lengths
    out, n, nodes = tn.inference_viterbi(links, u, tok, out_len, 2.5, 0.0, False, PAD)
    assert nodes == [[2]] and out.tolist() == [[8]]


def test_lookahead_case_worked_by_hand():
    p = torch.zeros(1, 5, 5)
    p[0, 0, 1] = .6; p[0, 0, 2] = .4; p[0, 1, 2] = .5; p[0, 1, 4] = .5; p[0, 2, 3] = .9; p[0, 2, 4] = .1; p[0, 3, 4] = 1.
    links = p.log()
    u = torch.tensor([[0.9, 0.1, 0.9, 0.8, 0.9]]).log()
    tok = torch.tensor([[5, 7, 8, 8, 2]])
    out_len = torch.tensor([5])
    # greedy: 0 -> 1 (.6); from 1 the two successors tie at .5: the lower node (2) wins; 2 -> 3 -> 4
    out, nodes = tn.inference_lookahead_simple(links, u, tok, out_len, 1.0, True, PAD)
    assert nodes == [[0, 1, 2, 3, 4]] and out.tolist() == [[5, 7, 8, 2]]           # 8 8 collapses
    # lookahead, beta 1: 0 -> 2 (.4 * .9 = .36 beats .6 * .1); 2 -> 3 (.9 * .8 beats .1 * .9); 3 -> 4
    out, nodes = tn.inference_lookahead_simple(links, u, tok, out_len, 1.0, False, PAD)
    assert nodes == [[0, 2, 3, 4]] and out.tolist() == [[5, 8, 2]]


@pytest.mark.parametrize("greedy", [False, True])
def test_lookahead_equals_loops_over_the_definition(greedy):
    import numpy as np
    B, L, beta = 5, 12, 0.7
    links, u, tok, out_len = decode_case(23, B, L)
    out, nodes = tn.inference_lookahead_simple(links, u, tok, out_len, beta, greedy, PAD)
    E, un = links.numpy(), u.numpy()
    for b in range(B):
        j, walk = 0, [0]
        while j != int(out_len[b]) - 1:
            score = [E[b, j, k] if greedy else np.float32(E[b, j, k] + np.float32(un[b, k] * np.float32(beta))) for k in range(L)]
            j = max(range(L), key=lambda k: (score[k], -k))                        # best score, lowest node among equals
            walk.append(j)
        assert nodes[b] == walk
        ys = [int(tok[b, x]) for x in walk]
        want = [y for k, y in enumerate(ys) if k == 0 or (y != PAD and y != ys[k - 1])]
        got = out[b].tolist()
        assert got[:len(want)] == want and all(t == PAD for t in got[len(want):])


def _golden():
    import os
    import numpy as np
    from conftest import ROOT
    return np.load(os.path.join(ROOT, "tests", "golden", "decode_small.npz"))


def test_oracle_reproduces_the_decoding_fixture():
    z = _golden()
    shifted = torch.from_numpy(z["links"]); u = torch.from_numpy(z["node_logp"]); tok = torch.from_numpy(z["node_tokens"])
    out_len = torch.from_numpy(z["out_len"]); pad = int(z["pad"])
    sq = tn.restore_valid_links(shifted)
    for key, joint in (("joint", True), ("plain", False)):
        tokens, n, nodes = tn.inference_viterbi(sq, u, tok, out_len, float(z["upsample_scale"]), float(z["viterbibeta"]), joint, pad)
        assert tokens.tolist() == z[f"viterbi_{key}_tokens"].tolist() and n.tolist() == z[f"viterbi_{key}_length"].tolist()
        assert [r + [-1] * (12 - len(r)) for r in nodes] == z[f"viterbi_{key}_nodes"].tolist()
    for key, greedy in (("lookahead", False), ("greedy", True)):
        tokens, nodes = tn.inference_lookahead_simple(sq, u, tok, out_len, float(z["decode_beta"]), greedy, pad)
        assert tokens.tolist() == z[f"{key}_tokens"].tolist()
        assert [r + [-1] * (24 - len(r)) for r in nodes] == z[f"{key}_nodes"].tolist()
