"""GPU parity of dag_multihead_links (through the C ABI) against the CPU oracle."""
import pytest
import torch

import da_transformer_amd as dagx
from oracle import torch_native as tn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NEG_INF = float("-inf")
# the kernels compute in fp32 and round once to the storage dtype
FWD_TOL = {torch.float32: (1e-5, 1e-5), torch.float16: (2e-3, 2e-3), torch.bfloat16: (1.6e-2, 1.6e-2)}
GRAD_RTOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 2e-2}


def _case(B, L, H, dtype, seed=0, scale=2.0, ragged=True):
    gen = torch.Generator().manual_seed(seed)
    content = (torch.randn(B, L, L, H, generator=gen) * scale).to(dtype)
    gates = torch.log_softmax(torch.randn(B, L, H, generator=gen), -1)
    if ragged:
        lens = torch.randint(2, L + 1, (B,), generator=gen)
        lens[0] = L
    else:
        lens = torch.full((B,), L)
    return content, gates, lens


def _mask(lens, L):
    return (torch.arange(L)[None, None, :] < lens[:, None, None]) & torch.ones(L, L, dtype=torch.bool).triu(1)[None]


def _compare(got, want, rtol, atol):
    finite = want > NEG_INF
    assert torch.equal(got > NEG_INF, finite), "different set of allowed transitions"
    assert not torch.isnan(got).any()
    assert torch.allclose(got[finite], want[finite], rtol=rtol, atol=atol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,translen", [(3, 17, 8, 5), (2, 70, 4, 100), (2, 300, 16, 64), (1, 1024, 8, 1023),
                                            (1, 600, 16, 599), (1, 1024, 16, 1023), (1, 498, 4, 497), (1, 786, 4, 785)])
def test_forward_and_backward_match_oracle(dtype, B, L, H, translen):
    content, gates, lens = _case(B, L, H, dtype)
    mask = _mask(lens, L)
    vend = lens[:, None].expand(-1, L).contiguous()
    # oracle in float64 on the same (rounded) inputs
    c64 = content.double().requires_grad_(); g64 = gates.double().requires_grad_()
    want = tn.multihead_links(c64, g64, mask, translen)
    weight = torch.randn(want.shape, generator=torch.Generator().manual_seed(5)).to(dtype)
    (want.masked_fill(want == NEG_INF, 0.0) * weight.double()).sum().backward()

    c = content.to(DEV).clone().requires_grad_(); g = gates.to(DEV).clone().requires_grad_()
    work = c * 1          # a non-leaf the operator may consume
    got = dagx.dag_multihead_links(work, g, vend.to(DEV), translen)
    assert got.dtype == dtype and got.shape == want.shape
    rtol, atol = FWD_TOL[dtype]
    _compare(got.detach().cpu().double(), want.detach(), rtol, atol)
    (got.masked_fill(got == NEG_INF, 0.0) * weight.to(DEV)).sum().backward()
    tol = GRAD_RTOL[dtype]
    for mine, ref in ((c.grad, c64.grad), (g.grad, g64.grad)):
        mine = mine.cpu().double()
        assert not torch.isnan(mine).any()
        assert torch.allclose(mine, ref, rtol=tol, atol=tol * ref.abs().max().item())
    # nothing outside the allowed transitions carries a gradient
    assert (c.grad.cpu()[~mask] == 0).all()


def test_bound_end_and_helpers():
    B, L, H = 2, 40, 8
    content, gates, _ = _case(B, L, H, torch.float32, seed=7, ragged=False)
    gen = torch.Generator().manual_seed(8)
    bound_end = torch.minimum(torch.arange(L)[None, :] + torch.randint(0, 9, (B, L), generator=gen), torch.tensor(L - 1))
    mask = (torch.arange(L)[None, None, :] <= bound_end[:, :, None]) & torch.ones(L, L, dtype=torch.bool).triu(1)[None]
    want = tn.multihead_links(content.double(), gates.double(), mask, 16)
    got = dagx.dag_multihead_links(content.to(DEV), gates.to(DEV), dagx.valid_end_from_bound(bound_end.to(DEV)), 16)
    _compare(got.cpu().double(), want, 1e-5, 1e-5)
    # decoder tokens with trailing padding
    pad = 1
    tokens = torch.full((B, L), 5); tokens[1, 30:] = pad
    vend = dagx.valid_end_from_tokens(tokens.to(DEV), pad)
    assert vend.shape == (B, L) and int(vend[0, 0]) == L and int(vend[1, 3]) == 30
    tokens[0, 4] = pad
    with pytest.raises(RuntimeError):
        dagx.valid_end_from_tokens(tokens.to(DEV), pad)


def test_feeds_dag_loss_and_extreme_scores():
    """The links go straight into dag_loss; huge score ranges and an all -inf head stay NaN-free."""
    B, L, H, T = 2, 64, 8, 9
    content, gates, lens = _case(B, L, H, torch.float32, seed=11, scale=30.0)
    content[0, 3, :, 2] = NEG_INF                      # head 2 of node 3 has no finite score
    mask = _mask(lens, L)
    vend = lens[:, None].expand(-1, L).contiguous()
    # (the reference's log_softmax turns such a head into NaN; here it simply drops out of the mixture,
    #  which the oracle reproduces with a -inf gate and harmless finite scores)
    c_ref = content.double().clone(); c_ref[0, 3, :, 2] = 0.0
    g_ref = gates.double().clone(); g_ref[0, 3, 2] = NEG_INF
    want = tn.multihead_links(c_ref, g_ref, mask, L - 1)
    got = dagx.dag_multihead_links(content.to(DEV), gates.to(DEV), vend.to(DEV), L - 1)
    _compare(got.cpu().double(), want, 1e-4, 1e-4)
    match = torch.log_softmax(torch.randn(B, T, L, generator=torch.Generator().manual_seed(2)), -1).to(DEV)
    tl = torch.tensor([T, 4]).to(DEV)
    ol = lens.clamp(min=T).to(DEV)
    vend2 = ol[:, None].expand(-1, L).contiguous()
    c = content.to(DEV).clamp(min=-100).requires_grad_()
    links = dagx.dag_multihead_links(c * 1, gates.to(DEV), vend2, L - 1)
    loss = dagx.dag_loss(match, links, ol, tl)
    loss.sum().backward()
    assert torch.isfinite(loss).all() and torch.isfinite(c.grad).all() and c.grad.abs().sum() > 0


def test_full_size_properties():
    """B=64, L=512, H=8 (the headline graph size): size-independent properties instead of the oracle.
    Every node with a successor gets a distribution over its transitions; the gradient of any function
    of the links sums to zero over a head's window (softmax) and the gate gradients sum to the incoming
    gradient mass of the node."""
    B, L, H = 64, 512, 8
    gen = torch.Generator(device=DEV).manual_seed(1)
    content = torch.randn(B, L, L, H, device=DEV, generator=gen) * 3
    gates = torch.log_softmax(torch.randn(B, L, H, device=DEV, generator=gen), -1).requires_grad_()
    lens = torch.randint(2, L + 1, (B,), device=DEV, generator=gen); lens[0] = L
    vend = lens[:, None].expand(-1, L).contiguous()
    c = content.requires_grad_()
    links = dagx.dag_multihead_links(c * 1, gates, vend, L - 1)
    total = torch.logsumexp(links.detach().float(), -1)                     # [B, L]
    has_next = torch.arange(L, device=DEV)[None, :] < (lens - 1)[:, None]
    assert torch.allclose(total[has_next], torch.zeros_like(total[has_next]), atol=2e-5)
    assert (total[~has_next] == NEG_INF).all()
    weight = torch.randn(links.shape, device=DEV, generator=gen)
    (links.masked_fill(links == NEG_INF, 0.0) * weight).sum().backward()
    assert torch.isfinite(c.grad).all() and torch.isfinite(gates.grad).all()
    per_head = c.grad.sum(2)                                                # sum over targets: [B, L, H]
    scale = c.grad.abs().sum(2).clamp(min=1.0)
    assert (per_head.abs() <= 1e-4 * scale).all()
    mass = (weight * (links.detach() > NEG_INF)).sum(-1)                    # incoming gradient of each node
    assert torch.allclose(gates.grad.sum(-1), mass, rtol=1e-4, atol=1e-3)


def test_argument_errors():
    c = torch.zeros(1, 8, 8, 3, device=DEV); g = torch.zeros(1, 8, 3, device=DEV)
    v = torch.full((1, 8), 8, device=DEV)
    with pytest.raises(RuntimeError, match="heads"):
        dagx.dag_multihead_links(c, g, v, 4)
    with pytest.raises(RuntimeError, match="valid_end"):
        dagx.dag_multihead_links(torch.zeros(1, 8, 8, 4, device=DEV), torch.zeros(1, 8, 4, device=DEV), v.int(), 4)


def test_scores_reused_after_backward_fail_loudly():
    """The backward writes the gradient over the scores; a node that had saved them for its own backward must
    raise rather than differentiate through gradient values."""
    B, L, H = 1, 40, 8
    content, gates, lens = _case(B, L, H, torch.float32, seed=3)
    vend = lens[:, None].expand(-1, L).contiguous().to(DEV)
    c = content.to(DEV).clone().requires_grad_()
    work = c * 1
    other_use = (work * work).sum()                    # saves `work` for its backward
    links = dagx.dag_multihead_links(work, gates.to(DEV), vend, L - 1)
    total = links.masked_fill(links == NEG_INF, 0.0).sum() + other_use
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        total.backward()
