"""GPU parity of dag_logsoftmax_gather_inplace (through the C ABI) against the CPU oracle."""
import os

import numpy as np
import pytest
import torch

import da_transformer_amd as dagx
from conftest import ROOT
from oracle import cref
from oracle import torch_native as tn
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# tolerances: the kernels accumulate in fp32 and round once to the storage dtype
SEL_RTOL, SEL_ATOL = 1e-4, 2e-5
GRAD_RTOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def _run_hip(logits, idx, gout=None):
    """logits: device tensor; returns (sel, grad or None).  The op sees a non-leaf, as in training."""
    if gout is None:
        same, sel = dagx.dag_logsoftmax_gather_inplace(logits, idx)
        assert same.data_ptr() == logits.data_ptr()
        return sel, None
    leaf = logits.clone().requires_grad_()
    work = leaf * 1                      # non-leaf copy the op may consume
    _, sel = dagx.dag_logsoftmax_gather_inplace(work, idx)
    (sel * gout).sum().backward()
    return sel.detach(), leaf.grad


def _oracle(logits_cpu, idx_cpu, gout_cpu=None):
    x = logits_cpu.float().requires_grad_(gout_cpu is not None)
    _, sel = tn.torch_dag_logsoftmax_gather_inplace(x, idx_cpu)
    if gout_cpu is None:
        return sel, None
    (sel * gout_cpu).sum().backward()
    return sel.detach(), x.grad


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("V", [37, 1000, 12347, 30522, 40000])
def test_forward_and_backward_match_oracle(dtype, V):
    B, L, S = 3, 5, 9
    c = workloads.gather_config(2, B=B, L=L, V=V, S=S, dtype=dtype)
    c["targets"][0, 1] = c["targets"][0, 0]         # a duplicated id in one sample
    idx = c["targets"].unsqueeze(1).expand(-1, L, -1)
    sel, grad = _run_hip(c["logits"].to(DEV), idx.to(DEV), c["grad_out"].to(DEV))
    rsel, rgrad = _oracle(c["logits"], idx, c["grad_out"])
    assert sel.dtype == torch.float32 and sel.shape == (B, L, S)
    assert torch.allclose(sel.cpu(), rsel, rtol=SEL_RTOL, atol=SEL_ATOL)
    tol = GRAD_RTOL[dtype]
    assert grad.dtype == dtype
    assert torch.allclose(grad.cpu().float(), rgrad, rtol=tol, atol=tol * rgrad.abs().max().item())
    # no-grad call leaves the logits untouched
    x = c["logits"].to(DEV)
    keep = x.clone()
    sel2, _ = _run_hip(x, idx.to(DEV))
    assert torch.equal(x, keep) and torch.equal(sel2, sel)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_transposed_storage_hands_over_a_contiguous_match(dtype):
    """selected stored as [B, S, L]: same values, its transpose is the contiguous [B, T, L] tensor the
    criterion feeds to dag_loss (nat_dag_loss.py:169), and the gradient flows back through both ops
    exactly as with the default storage."""
    B, L, S, V = 3, 70, 9, 1234
    c = workloads.gather_config(2, B=B, L=L, V=V, S=S, dtype=dtype)
    idx = c["targets"].unsqueeze(1).expand(-1, L, -1).to(DEV)
    gen = torch.Generator().manual_seed(3)
    links = torch.log_softmax(torch.randn(B, L, L - 1, generator=gen), -1).to(DEV)
    links = links.masked_fill(torch.arange(L, device=DEV)[None, :, None] + torch.arange(L - 1, device=DEV)[None, None, :] + 1 >= L, float("-inf"))
    ol = torch.tensor([L, L - 7, L - 30], device=DEV); tl = torch.tensor([S, S - 2, 4], device=DEV)

    def run(transposed):
        leaf = c["logits"].to(DEV).clone().requires_grad_()
        lk = links.clone().requires_grad_()
        _, sel = dagx.dag_logsoftmax_gather_inplace(leaf * 1, idx, transposed)
        match = sel.transpose(1, 2)
        loss = dagx.dag_loss(match, lk, ol, tl)
        loss.sum().backward()
        return sel.detach(), match.is_contiguous(), loss.detach(), leaf.grad, lk.grad

    sel0, contig0, loss0, g0, gl0 = run(False)
    sel1, contig1, loss1, g1, gl1 = run(True)
    assert not contig0 and contig1
    assert sel1.shape == (B, L, S) and torch.equal(sel0, sel1)
    assert torch.allclose(loss0, loss1, rtol=1e-6, atol=0)
    tol = GRAD_RTOL[dtype]
    assert torch.allclose(g0.float(), g1.float(), rtol=tol, atol=tol * g0.float().abs().max().item())
    assert torch.allclose(gl0, gl1, rtol=1e-5, atol=1e-7)
    # and against the oracle
    rsel, _ = _oracle(c["logits"], idx.cpu())
    assert torch.allclose(sel1.cpu(), rsel, rtol=SEL_RTOL, atol=SEL_ATOL)


def test_contiguous_index_and_misaligned_rows():
    """Independent ids per row (contiguous index) and a row pitch that is not a multiple of 16 bytes."""
    g = torch.Generator().manual_seed(5)
    B, L, V, S = 2, 7, 2001, 33
    x = (torch.randn(B, L, V, generator=g) * 3).half()
    idx = torch.randint(0, V, (B, L, S), generator=g)
    idx[1, 2, :5] = idx[1, 2, 7]                     # heavy duplication inside one row
    gout = torch.randn(B, L, S, generator=g)
    sel, grad = _run_hip(x.to(DEV), idx.to(DEV), gout.to(DEV))
    rsel, rgrad = _oracle(x, idx, gout)
    assert torch.allclose(sel.cpu(), rsel, rtol=SEL_RTOL, atol=SEL_ATOL)
    assert torch.allclose(grad.cpu().float(), rgrad, rtol=1e-2, atol=1e-2 * rgrad.abs().max().item())
    # exact properties of the result: every row of the gradient sums to ~0 in fp32 terms
    rows = grad.cpu().float().sum(-1)
    assert rows.abs().max() < 0.05


def test_golden_fixture():
    z = np.load(os.path.join(ROOT, "tests", "golden", "gather_small.npz"))
    logits = torch.from_numpy(z["logits"])
    idx = torch.from_numpy(z["targets"]).unsqueeze(1).expand(-1, logits.shape[1], -1)
    sel, grad = _run_hip(logits.to(DEV), idx.to(DEV), torch.from_numpy(z["grad_out"]).to(DEV))
    assert np.allclose(sel.cpu().numpy().reshape(z["sel"].shape), z["sel"], rtol=SEL_RTOL, atol=SEL_ATOL)
    ref = z["grad_logits"].reshape(grad.shape)
    assert np.allclose(grad.cpu().numpy(), ref, rtol=1e-4, atol=1e-4 * np.abs(ref).max())


def test_masked_logits_and_extreme_values():
    x = torch.randn(1, 4, 515) * 20
    x[0, 0, 100:200] = float("-inf")                 # masked vocabulary entries
    x[0, 1, 3] = 80.0                                # one dominant logit
    idx = torch.tensor([[[0, 3, 150, 514]]]).expand(1, 4, 4)
    sel, _ = _run_hip(x.to(DEV), idx.to(DEV))
    rsel, _ = _oracle(x, idx)
    fin = torch.isfinite(rsel)
    assert torch.equal(torch.isfinite(sel.cpu()), fin)
    assert torch.allclose(sel.cpu()[fin], rsel[fin], rtol=SEL_RTOL, atol=SEL_ATOL)


def test_empty_batch_and_no_ids():
    x = torch.randn(0, 4, 33, device=DEV); idx = torch.zeros(0, 4, 3, dtype=torch.long, device=DEV)
    assert dagx.dag_logsoftmax_gather_inplace(x, idx)[1].shape == (0, 4, 3)
    x = torch.randn(2, 3, 50, device=DEV); idx = torch.zeros(2, 3, 0, dtype=torch.long, device=DEV)
    assert dagx.dag_logsoftmax_gather_inplace(x, idx)[1].shape == (2, 3, 0)
    leaf = x.clone().requires_grad_()
    _, sel = dagx.dag_logsoftmax_gather_inplace(leaf * 1, idx)
    sel.sum().backward()
    assert (leaf.grad == 0).all()


def test_api_contract():
    x = torch.randn(2, 3, 50, device=DEV)
    idx = torch.randint(0, 50, (2, 3, 4), device=DEV)
    with pytest.raises(RuntimeError):
        dagx.dag_logsoftmax_gather_inplace(x.transpose(0, 1), idx.transpose(0, 1))   # not contiguous
    with pytest.raises(RuntimeError):
        dagx.dag_logsoftmax_gather_inplace(x, idx.int())
    # a leaf that requires grad cannot be consumed in place (same as the reference)
    with pytest.raises(RuntimeError):
        dagx.dag_logsoftmax_gather_inplace(x.clone().requires_grad_(), idx)
    # backward twice is refused
    leaf = x.clone().requires_grad_()
    _, sel = dagx.dag_logsoftmax_gather_inplace(leaf * 1, idx)
    sel.sum().backward(retain_graph=True)
    with pytest.raises(AssertionError):
        sel.sum().backward()


def test_full_size_properties():
    """[64,512,40000] fp16: checked on a row sample against the float64 C oracle and through
    size-independent properties (probabilities of a row sum to 1; gradient rows sum to 0)."""
    c = workloads.gather_config(2, device=DEV)
    x, idx, gout = c["logits"], c["select_idx"], c["grad_out"]
    rows = torch.tensor([0, 1, 511, 512, 20000, 32767])
    x_rows = x.view(-1, c["V"])[rows.to(DEV)].cpu()
    sel, _ = _run_hip(x, idx)
    want, lse = cref.lsg(x_rows.double().numpy(), idx.reshape(-1, c["S"])[rows.to(DEV)].cpu().numpy())
    got = sel.view(-1, c["S"])[rows.to(DEV)].cpu().numpy()
    assert np.allclose(got, want, rtol=SEL_RTOL, atol=SEL_ATOL)
    # backward, in place on a scratch copy (non-leaf path)
    leaf = x.clone().requires_grad_()
    _, sel2 = dagx.dag_logsoftmax_gather_inplace(leaf * 1, idx)
    (sel2 * gout).sum().backward()
    grad = leaf.grad
    g_rows = grad.view(-1, c["V"])[rows.to(DEV)].cpu().double().numpy()
    ref = cref.lsg_bwd(x_rows.double().numpy(), idx.reshape(-1, c["S"])[rows.to(DEV)].cpu().numpy(),
                       gout.reshape(-1, c["S"])[rows.to(DEV)].cpu().double().numpy())
    assert np.allclose(g_rows, ref, rtol=1e-2, atol=1e-2 * np.abs(ref).max())
    sums = grad.float().sum(-1)
    assert sums.abs().max().item() < 0.25            # fp16 rounding of 40000 entries per row


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("V", [37, 1000, 12347, 40000])
@pytest.mark.parametrize("ties", [False, True])
def test_argmax_in_the_same_pass(dtype, V, ties):
    """pred_tokens = word_ins_out.argmax(-1) (nat_dag_loss.py:246) out of the gather's own pass:
    bit-exact indices (first index among equal logits), identical gathered values."""
    gen = torch.Generator().manual_seed(V + int(ties))
    B, L, S = 2, 9, 5                                   # odd V: most rows start off a 16-byte boundary
    x = torch.randn(B, L, V, generator=gen) * 3
    if ties:
        x = (x * 2).round() / 8                         # a coarse grid: the row maximum repeats
        x[0, 0] = 0.0                                   # a whole row ties: index 0
        x[0, 1, :] = -1.0; x[0, 1, V - 1] = 2.0; x[0, 1, V // 2] = 2.0     # tail element against the vector stream
        x[0, 2] = float("-inf")                         # arg max of a row of -inf is 0
    x = x.to(dtype)
    idx = torch.randint(0, V, (B, L, S), generator=gen)
    dev = x.to(DEV)
    _, sel, pred = dagx.dag_logsoftmax_gather_argmax(dev, idx.to(DEV))
    assert torch.equal(pred.cpu(), x.float().argmax(-1))
    _, sel_plain = dagx.dag_logsoftmax_gather_inplace(dev, idx.to(DEV))
    assert torch.equal(sel.cpu().view(torch.int32), sel_plain.cpu().view(torch.int32))
    values, tokens = dagx.dag_logsoftmax_max(dev)
    want_values, want_tokens = x.float().log_softmax(-1).max(-1)
    assert torch.equal(tokens.cpu(), want_tokens)
    finite = torch.isfinite(want_values)
    assert torch.allclose(values.cpu()[finite], want_values[finite], rtol=SEL_RTOL, atol=SEL_ATOL)


def test_argmax_full_size():
    """[64,512,40000] fp16: the arg max of every row against torch on the same device."""
    x = workloads.gather_config(2, device=DEV)["logits"]
    values, tokens = dagx.dag_logsoftmax_max(x)
    # fp16 rows repeat their maximum now and then: compare values at the indices, and the index rule on ties
    assert torch.equal(x.gather(-1, tokens.unsqueeze(-1)).squeeze(-1), x.max(-1).values)
    first = (x == x.max(-1, keepdim=True).values).int().argmax(-1)            # first position of the maximum
    assert torch.equal(tokens, first)
    rows = slice(0, 4)
    want = x[rows].float().log_softmax(-1).max(-1).values
    assert torch.allclose(values[rows], want, rtol=SEL_RTOL, atol=SEL_ATOL)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_one_dominant_logit_at_every_slot_of_a_vector(dtype):
    """The running maximum that keeps the exponentials in range must see every element of a 16-byte
    vector: one logit far above the rest (exp of the gap overflows fp32), at each of 16 positions."""
    V, big = 4096, 120.0
    x = torch.zeros(1, 16, V)
    for pos in range(16):
        x[0, pos, 1024 + pos] = big
    x = x.to(dtype)
    idx = (1024 + torch.arange(16)).view(1, 16, 1).repeat(1, 1, 2)
    idx[:, :, 1] = 0
    sel, _ = _run_hip(x.to(DEV), idx.to(DEV))
    want, _ = _oracle(x, idx)
    assert torch.isfinite(sel).all()
    assert torch.allclose(sel.cpu(), want, rtol=SEL_RTOL, atol=SEL_ATOL)
    values, tokens = dagx.dag_logsoftmax_max(x.to(DEV))
    assert torch.equal(tokens.cpu(), idx[:, :, 0])


@pytest.mark.parametrize("V,S,dtype", [(2001, 300, torch.float16), (30522, 256, torch.float16), (40000, 512, torch.float32),
                                       (12347, 128, torch.bfloat16), (2000001, 128, torch.float16), (999, 96, torch.float32),
                                       (5000, 4096, torch.float32)])   # the documented maximum of ids per row
def test_many_gathered_ids_per_row(V, S, dtype):
    """Rows with a hundred and more gathered ids take the backward's other route (scatter terms added
    inside the stream, duplicates found through a hash table); a vocabulary whose bitmap does not fit
    falls back.  Ids repeat two-, three- and many-fold, per row independently."""
    g = torch.Generator().manual_seed(V + S)
    B, L = 2, 3
    x = (torch.randn(B, L, V, generator=g) * 3).to(dtype)
    pool = torch.randint(0, V, (B, L, max(S // 3, 1)), generator=g)         # few distinct ids -> many duplicates
    idx = pool.gather(-1, torch.randint(0, pool.shape[-1], (B, L, S), generator=g))
    idx[0, 0] = torch.randperm(V, generator=g)[:S] if V >= S else idx[0, 0]  # one row without any duplicate
    idx[0, 1] = idx[0, 1, 0]                                                 # one row with a single id
    gout = torch.randn(B, L, S, generator=g)
    sel, grad = _run_hip(x.to(DEV), idx.to(DEV), gout.to(DEV))
    rsel, rgrad = _oracle(x, idx, gout)
    assert torch.allclose(sel.cpu(), rsel, rtol=SEL_RTOL, atol=SEL_ATOL)
    tol = GRAD_RTOL[dtype]
    assert torch.allclose(grad.cpu().float(), rgrad, rtol=tol, atol=tol * rgrad.abs().max().item())
    # transposed incoming gradient (the criterion's form) gives the same bits
    _, grad_t = _run_hip(x.detach().to(DEV), idx.to(DEV), gout.transpose(1, 2).contiguous().transpose(1, 2).to(DEV))
    assert torch.equal(grad_t, grad)


@pytest.mark.parametrize("S", [8, 200])
def test_ids_outside_the_vocabulary_give_nan_and_no_gradient(S):
    """With few and with many ids per row (the backward has a route for each)."""
    g = torch.Generator().manual_seed(S)
    B, L, V = 1, 2, 20000
    x = torch.randn(B, L, V, generator=g).half()
    idx = torch.randint(0, V, (B, L, S), generator=g)
    idx[0, 0, 1] = -1; idx[0, 1, 3] = V; idx[0, 1, 5] = idx[0, 1, 4]
    bad = torch.zeros(B, L, S, dtype=torch.bool); bad[0, 0, 1] = True; bad[0, 1, 3] = True
    gout = torch.randn(B, L, S, generator=g)
    sel, grad = _run_hip(x.to(DEV), idx.to(DEV), gout.masked_fill(bad, 0.0).to(DEV))
    assert torch.equal(torch.isnan(sel.cpu()), bad)
    rsel, rgrad = _oracle(x, idx.clamp(0, V - 1), gout.masked_fill(bad, 0.0))
    assert torch.allclose(sel.cpu()[~bad], rsel[~bad], rtol=SEL_RTOL, atol=SEL_ATOL)
    assert torch.allclose(grad.cpu().float(), rgrad, rtol=1e-2, atol=1e-2 * rgrad.abs().max().item())
