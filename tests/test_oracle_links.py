"""Pins oracle.torch_native.multihead_links (the restated tail of extract_links,
glat_decomposed_with_link.py:319-335, 380-404) without running the reference."""
import math

import pytest
import torch

from oracle import torch_native as tn

NEG_INF = float("-inf")


def _case(B=3, L=9, H=4, seed=0, dtype=torch.float64):
    gen = torch.Generator().manual_seed(seed)
    content = torch.randn(B, L, L, H, generator=gen, dtype=dtype) * 2
    gates = torch.log_softmax(torch.randn(B, L, H, generator=gen, dtype=dtype), -1)
    lens = torch.tensor([L, L - 3, 2][:B])
    upper = torch.ones(L, L, dtype=torch.bool).triu(1)
    mask = (torch.arange(L)[None, None, :] < lens[:, None, None]) & upper[None]
    return content, gates, mask, lens


def _loops(content, gates, mask, translen):
    """The definition, element by element in float64."""
    B, L, _, H = content.shape
    translen = min(translen, L - 1)
    out = torch.full((B, L, translen), NEG_INF, dtype=torch.float64)
    for b in range(B):
        for i in range(L):
            if not mask[b, i].any():
                continue
            win = [j for j in range(i + 1, min(L, i + 1 + translen)) if mask[b, i, j]]
            for j in win:
                tot = 0.0
                for c in range(H):
                    z = sum(math.exp(float(content[b, i, jj, c])) for jj in win)
                    tot += math.exp(float(gates[b, i, c]) + float(content[b, i, j, c]) - math.log(z))
                out[b, i, j - i - 1] = math.log(tot)
    return out


@pytest.mark.parametrize("translen", [3, 8, 100])
def test_matches_elementwise_definition(translen):
    content, gates, mask, _ = _case()
    got = tn.multihead_links(content, gates, mask, translen)
    want = _loops(content, gates, mask, translen)
    assert got.shape == want.shape
    finite = want > NEG_INF
    assert torch.equal(got > NEG_INF, finite)
    assert torch.allclose(got[finite], want[finite], rtol=1e-12, atol=1e-12)


def test_rows_are_distributions_and_one_head_is_log_softmax():
    content, gates, mask, lens = _case(H=4)
    links = tn.multihead_links(content, gates, mask, 100)
    total = torch.logsumexp(links, -1)
    for b in range(content.shape[0]):
        n = int(lens[b])
        assert torch.allclose(total[b, :n - 1], torch.zeros(n - 1, dtype=torch.float64), atol=1e-12)
        assert (total[b, n - 1:] == NEG_INF).all()          # the last node and the padding have no transition
    one = content[..., :1]
    zero_gate = torch.zeros_like(gates[..., :1])
    links1 = tn.multihead_links(one, zero_gate, mask, 100)
    square = one[..., 0].masked_fill(~mask, NEG_INF)
    ref = tn.extract_valid_links(torch.log_softmax(square, -1).nan_to_num(nan=NEG_INF, neginf=NEG_INF))
    assert torch.allclose(links1.nan_to_num(neginf=-1e30), ref.nan_to_num(neginf=-1e30), atol=1e-12)


def test_bound_end_mask_and_gradcheck():
    content, gates, _, _ = _case(B=2, L=6, H=4, seed=3)
    L = content.shape[1]
    bound_end = torch.tensor([[2, 3, 3, 5, 5, 5], [1, 1, 4, 4, 5, 5]])
    mask = (torch.arange(L)[None, None, :] <= bound_end[:, :, None]) & torch.ones(L, L, dtype=torch.bool).triu(1)[None]
    want = _loops(content, gates, mask, 4)
    got = tn.multihead_links(content, gates, mask, 4)
    finite = want > NEG_INF
    assert torch.equal(got > NEG_INF, finite) and torch.allclose(got[finite], want[finite], atol=1e-12)
    c = content.clone().requires_grad_(); g = gates.clone().requires_grad_()
    weight = torch.randn(got.shape, dtype=torch.float64, generator=torch.Generator().manual_seed(1))

    def f(c_, g_):
        out = tn.multihead_links(c_, g_, mask, 4)
        return (out.masked_fill(~finite, 0.0) * weight).sum()
    assert torch.autograd.gradcheck(f, (c, g), atol=1e-8)
