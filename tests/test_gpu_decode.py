"""GPU parity of dag_viterbi_decode and dag_lookahead_decode (through the C ABI) against the CPU oracle: predicted length,
the path's nodes and the collapsed tokens, bit for bit -- including inputs full of ties, where the
first-index rule of the tensor formulation decides."""
import pytest
import torch

import da_transformer_amd as dagx
from da_transformer_amd import _native as nat
from oracle import torch_native as tn
from test_oracle_viterbi import decode_case, PAD

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def peaked_case(seed, B, L, hop=4, vocab=50, min_len=128):
    """Graphs whose transitions favour i -> i + hop, so that long paths win (as a trained model's do)."""
    gen = torch.Generator().manual_seed(seed)
    out_len = torch.randint(min_len, L + 1, (B,), generator=gen)
    out_len[0] = L
    i = torch.arange(L).view(1, L, 1); j = torch.arange(L).view(1, 1, L)
    logits = torch.randn(B, L, L, generator=gen) + 8.0 * (j == i + hop)
    ok = (j > i) & (j < out_len.view(B, 1, 1))
    logits = logits.masked_fill(~ok, float("-inf"))
    dead = ~ok.any(-1, keepdim=True)
    links = torch.log_softmax(logits.masked_fill(dead, 0.0), -1).masked_fill(~ok, float("-inf"))
    u, tok = torch.log_softmax(torch.randn(B, L, vocab, generator=gen) * 2, -1).max(-1)
    return links, u, tok, out_len


def _run_and_compare(links_sq, u, tok, out_len, translen, scale, beta, joint, dtype=torch.float32):
    B, L = u.shape
    shifted = tn.extract_valid_links(links_sq, translen).to(dtype)
    square = tn.restore_valid_links(shifted.float())           # what the kernel's input means
    want_tokens, want_len, want_nodes = tn.inference_viterbi(square, u, tok, out_len, scale, beta, joint, PAD)
    got = dagx.dag_viterbi_decode(shifted.to(DEV), (u.to(DEV), tok.to(DEV)), out_len.to(DEV), scale, beta, joint, PAD)
    assert torch.equal(got.pred_length.cpu(), want_len)
    nodes = got.nodes.cpu()
    for b in range(B):
        n = int(want_len[b])
        assert nodes[b, :n].tolist() == want_nodes[b], f"sample {b}"
        assert (nodes[b, n:] == -1).all()
    assert not got.output_tokens.is_cuda and got.output_tokens.dtype == torch.int64
    assert torch.equal(got.output_tokens, want_tokens)
    assert got.output_scores.shape == want_tokens.shape and (got.output_scores == 1).all()


@pytest.mark.parametrize("joint", [False, True])
@pytest.mark.parametrize("B,L,translen,scale,beta", [
    (6, 9, 8, 3.0, 1.0), (5, 40, 39, 4.0, 0.0), (3, 130, 50, 4.0, 1.0), (4, 300, 299, 8.0, 0.5), (2, 1024, 1023, 16.0, 1.0)])
def test_viterbi_decode_matches_the_oracle(B, L, translen, scale, beta, joint):
    links, u, tok, out_len = decode_case(100 + L, B, L, vocab=7)
    out_len[-1] = 2 if L < 100 else 3                        # a graph with (next to) no interior node
    links = links.masked_fill(torch.arange(L).view(1, 1, L) >= out_len.view(B, 1, 1), float("-inf"))
    _run_and_compare(links, u, tok, out_len, translen, scale, beta, joint)


@pytest.mark.parametrize("joint", [False, True])
def test_viterbi_decode_full_size(joint):
    """B=64, L=512 (64 source tokens upsampled 8 times), 128 steps."""
    links, u, tok, out_len = peaked_case(5, 64, 512)
    _run_and_compare(links, u, tok, out_len, 511, 8.0, 1.0, joint)
    links, u, tok, out_len = decode_case(5, 64, 512, vocab=50, min_len=128)
    _run_and_compare(links, u, tok, out_len, 511, 8.0, 1.0, joint)


@pytest.mark.parametrize("joint", [False, True])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_viterbi_decode_ties(joint, beta):
    """Scores on a coarse grid: many predecessors, last nodes and lengths tie exactly."""
    B, L = 6, 70
    links, u, tok, out_len = decode_case(9, B, L, vocab=4)
    links = (links * 2).round() / 2
    u = (u * 2).round() / 2
    _run_and_compare(links, u, tok, out_len, L - 1, 4.0, beta, joint)
    flat = torch.where(torch.isfinite(links), torch.zeros_like(links), links)    # every transition equal
    _run_and_compare(flat, torch.zeros_like(u), tok, out_len, L - 1, 4.0, beta, joint)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_viterbi_decode_half_precision_links(dtype):
    links, u, tok, out_len = decode_case(31, 4, 90, vocab=9)
    _run_and_compare(links, u, tok, out_len, 60, 4.0, 1.0, True, dtype=dtype)


def test_viterbi_decode_one_workgroup_route():
    """The route taken by samples the pipeline gives up on (forced for every sample here)."""
    links, u, tok, out_len = decode_case(41, 5, 150, vocab=9)
    before = nat.lib().dagx_force_log_domain(1)
    try:
        _run_and_compare(links, u, tok, out_len, 149, 4.0, 1.0, True)
        _run_and_compare(links, u, tok, out_len, 40, 4.0, 0.0, False)
        flat = torch.where(torch.isfinite(links), torch.zeros_like(links), links)    # every transition equal
        _run_and_compare(flat, torch.zeros_like(u), tok, out_len, 149, 4.0, 1.0, True)
        links, u, tok, out_len = decode_case(42, 3, 400, vocab=9)
        _run_and_compare(links, u, tok, out_len, 399, 4.0, 1.0, True, dtype=torch.float16)
    finally:
        nat.lib().dagx_force_log_domain(before)


def test_viterbi_decode_takes_the_logits_tensor_and_checks_arguments():
    links, u, tok, out_len = decode_case(51, 3, 30, vocab=11)
    gen = torch.Generator().manual_seed(1)
    logits = torch.log_softmax(torch.randn(3, 30, 11, generator=gen), -1)
    u2, tok2 = logits.max(-1)
    shifted = tn.extract_valid_links(links)
    want = tn.inference_viterbi(tn.restore_valid_links(shifted), u2, tok2, out_len, 3.0, 1.0, True, PAD)[0]
    got = dagx.dag_viterbi_decode(shifted.to(DEV), logits.to(DEV), out_len.to(DEV), 3.0, 1.0, True, PAD)
    assert torch.equal(got.output_tokens, want)
    with pytest.raises(RuntimeError):
        dagx.dag_viterbi_decode(shifted.to(DEV), logits[:, :5].to(DEV), out_len.to(DEV), 3.0, 1.0, True, PAD)
    with pytest.raises(RuntimeError):
        dagx.dag_viterbi_decode(shifted.to(DEV), logits.to(DEV), out_len.int().to(DEV), 3.0, 1.0, True, PAD)
    with pytest.raises(RuntimeError):
        dagx.dag_viterbi_decode(shifted, logits, out_len, 3.0, 1.0, True, PAD)


def _walk_and_compare(links_sq, u, tok, out_len, translen, beta, greedy, dtype=torch.float32):
    B, L = u.shape
    shifted = tn.extract_valid_links(links_sq, translen).to(dtype)
    square = tn.restore_valid_links(shifted.float())
    want_tokens, want_nodes = tn.inference_lookahead_simple(square, u, tok, out_len, beta, greedy, PAD)
    got = dagx.dag_lookahead_decode(shifted.to(DEV), (u.to(DEV), tok.to(DEV)), out_len.to(DEV), beta, greedy, PAD)
    nodes = got.nodes.cpu()
    for b in range(B):
        n = len(want_nodes[b])
        assert nodes[b, :n].tolist() == want_nodes[b], f"sample {b}"
        assert (nodes[b, n:] == -1).all()
    assert not got.output_tokens.is_cuda and torch.equal(got.output_tokens, want_tokens)
    assert (got.output_scores == 1).all() and got.output_scores.shape == want_tokens.shape


@pytest.mark.parametrize("greedy", [False, True])
@pytest.mark.parametrize("B,L,translen,beta", [(6, 9, 8, 1.0), (5, 40, 39, 0.3), (3, 130, 50, 1.0), (64, 512, 511, 1.0), (2, 1500, 700, 1.0)])
def test_lookahead_decode_matches_the_oracle(B, L, translen, beta, greedy):
    links, u, tok, out_len = decode_case(200 + L, B, L, vocab=7)
    out_len[-1] = 1 if L < 100 else 2                        # graphs without an interior node
    links = links.masked_fill(torch.arange(L).view(1, 1, L) >= out_len.view(B, 1, 1), float("-inf"))
    _walk_and_compare(links, u, tok, out_len, translen, beta, greedy)


@pytest.mark.parametrize("greedy", [False, True])
def test_lookahead_decode_ties_and_half_precision(greedy):
    links, u, tok, out_len = decode_case(13, 6, 70, vocab=4)
    _walk_and_compare((links * 2).round() / 2, (u * 2).round() / 2, tok, out_len, 69, 1.0, greedy)
    flat = torch.where(torch.isfinite(links), torch.zeros_like(links), links)      # every successor ties: node i+1 wins
    _walk_and_compare(flat, torch.zeros_like(u), tok, out_len, 69, 1.0, greedy)
    _walk_and_compare(links, u, tok, out_len, 30, 0.5, greedy, dtype=torch.float16)
    _walk_and_compare(links, u, tok, out_len, 30, 0.5, greedy, dtype=torch.bfloat16)


def test_lookahead_decode_stops_on_a_graph_without_a_way_out():
    """A row of -inf sends the walk back to node 0 (the arg max of the tensor formulation, which then
    never returns); the kernel stops after prelen nodes."""
    links, u, tok, out_len = decode_case(17, 2, 20, vocab=5)
    links[1, 0] = float("-inf")
    got = dagx.dag_lookahead_decode(tn.extract_valid_links(links).to(DEV), (u.to(DEV), tok.to(DEV)), out_len.to(DEV), 1.0, False, PAD)
    assert (got.nodes[1].cpu() == 0).all()
    assert got.output_tokens[1, 0] == tok[1, 0]


def test_decoding_golden_fixture():
    import os
    import numpy as np
    from conftest import ROOT
    z = np.load(os.path.join(ROOT, "tests", "golden", "decode_small.npz"))
    links = torch.from_numpy(z["links"]).to(DEV); u = torch.from_numpy(z["node_logp"]).to(DEV)
    tok = torch.from_numpy(z["node_tokens"]).to(DEV); out_len = torch.from_numpy(z["out_len"]).to(DEV); pad = int(z["pad"])
    for key, joint in (("joint", True), ("plain", False)):
        r = dagx.dag_viterbi_decode(links, (u, tok), out_len, float(z["upsample_scale"]), float(z["viterbibeta"]), joint, pad)
        assert r.output_tokens.tolist() == z[f"viterbi_{key}_tokens"].tolist()
        assert r.pred_length.cpu().tolist() == z[f"viterbi_{key}_length"].tolist()
        assert r.nodes.cpu().tolist() == z[f"viterbi_{key}_nodes"].tolist()
    for key, greedy in (("lookahead", False), ("greedy", True)):
        r = dagx.dag_lookahead_decode(links, (u, tok), out_len, float(z["decode_beta"]), greedy, pad)
        assert r.output_tokens.tolist() == z[f"{key}_tokens"].tolist()
        assert r.nodes.cpu().tolist() == z[f"{key}_nodes"].tolist()
