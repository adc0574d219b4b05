"""Writes tests/golden/*.npz: inputs and expected outputs of small seeded cases, computed by the
CPU oracle (float64 C restatement for the loss and its gradients, float32 torch restatement for
the alignment).  Run from the repository root:  python tests/golden/make_fixtures.py
The reference ships no vectors for this path, so these come from the pinned oracle."""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import cref                      # noqa: E402
from oracle import torch_native as tn        # noqa: E402
import workloads                             # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def dag_case(name, cfg):
    match, links = cfg["match"].float(), cfg["links"].float()
    sq = tn.restore_valid_links(links)
    ol, tl, g = cfg["out_len"], cfg["tgt_len"], cfg["grad_out"]
    loss, gm, gl_sq = cref.dag_loss_grad(match.numpy(), sq.numpy(), ol.numpy(), tl.numpy(), g.numpy())
    gl = tn.extract_valid_links(torch.from_numpy(gl_sq), links.shape[2])
    gl = gl.masked_fill(torch.isinf(gl), 0.0).numpy()
    path = tn.torch_dag_best_alignment(match, sq, ol, tl).numpy()
    np.savez_compressed(os.path.join(HERE, name), match=cfg["match"].numpy(), links=cfg["links"].numpy(),
                        out_len=ol.numpy(), tgt_len=tl.numpy(), grad_out=g.numpy(),
                        loss=loss, grad_match=gm.astype(np.float32), grad_links=gl.astype(np.float32), path=path)


def gather_case(name):
    c = workloads.gather_config(2, B=2, L=8, V=1003, S=12, dtype=torch.float32)
    x = c["logits"].view(-1, 1003).double().numpy()
    idx = c["select_idx"].contiguous().view(-1, 12).numpy()
    g = c["grad_out"].contiguous().view(-1, 12).double().numpy()
    sel, lse = cref.lsg(x, idx)
    gx = cref.lsg_bwd(x, idx, g)
    np.savez_compressed(os.path.join(HERE, name), logits=c["logits"].numpy(), targets=c["targets"].numpy(),
                        grad_out=c["grad_out"].contiguous().numpy(), sel=sel.astype(np.float32),
                        lse=lse.astype(np.float32), grad_logits=gx.astype(np.float32))


def _pad_lists(rows, width, fill=-1):
    return np.array([r + [fill] * (width - len(r)) for r in rows], dtype=np.int64)


def decode_case(name):
    """Graph decoding: Viterbi (joint and plain, beta 1) and the lookahead / greedy walks on one small batch."""
    from test_oracle_viterbi import decode_case as make, PAD
    links_sq, u, tok, out_len = make(77, 5, 24, vocab=9)
    shifted = tn.extract_valid_links(links_sq, 15)
    sq = tn.restore_valid_links(shifted)
    out = dict(links=shifted.numpy(), node_logp=u.numpy(), node_tokens=tok.numpy(), out_len=out_len.numpy(), pad=np.int64(PAD),
               upsample_scale=np.float64(4.0), viterbibeta=np.float64(1.0), decode_beta=np.float64(1.0))
    for key, joint in (("joint", True), ("plain", False)):
        tokens, n, nodes = tn.inference_viterbi(sq, u, tok, out_len, 4.0, 1.0, joint, PAD)
        out[f"viterbi_{key}_tokens"] = tokens.numpy(); out[f"viterbi_{key}_length"] = n.numpy()
        out[f"viterbi_{key}_nodes"] = _pad_lists(nodes, 12)
    for key, greedy in (("lookahead", False), ("greedy", True)):
        tokens, nodes = tn.inference_lookahead_simple(sq, u, tok, out_len, 1.0, greedy, PAD)
        out[f"{key}_tokens"] = tokens.numpy(); out[f"{key}_nodes"] = _pad_lists(nodes, 24)
    np.savez_compressed(os.path.join(HERE, name), **out)


def glance_case(name):
    """Glancing glue and force-emit on one small batch."""
    from test_oracle_glat import random_case
    path, tgt, pred, prev, mask, tgt_len, rand = random_case(5, B=4, L=20, T=8, vocab=30)
    oracle, same, kp, keep, tokens, force = tn.glat_glance(path, tgt, pred, prev, mask, tgt_len, 0.5, rand)
    gen = torch.Generator().manual_seed(9)
    match = torch.randn(4, 8, 20, generator=gen)
    np.savez_compressed(os.path.join(HERE, name), path=path.numpy(), tgt_tokens=tgt.numpy(), pred_tokens=pred.numpy(),
                        prev_output_tokens=prev.numpy(), prev_mask=mask.numpy(), tgt_len=tgt_len.numpy(), rand=rand.numpy(),
                        context_p=np.float64(0.5), oracle=oracle.numpy(), same_num=same.numpy(), keep_prob=kp.numpy(),
                        keep_word_mask=keep.numpy(), glat_prev_output_tokens=tokens.numpy(), next_force_emit=force.numpy(),
                        match=match.numpy(), forced_match=tn.force_alignment(match, force).numpy())


if __name__ == "__main__":
    decode_case("decode_small.npz")
    glance_case("glance_small.npz")
    dag_case("dag_cfg0.npz", workloads.dag_config(0))
    ragged = workloads.dag_config(0, translen=20)
    ragged["out_len"] = torch.tensor([64, 50, 33, 17]); ragged["tgt_len"] = torch.tensor([16, 9, 16, 2])
    # rows beyond L_b keep stale finite values on purpose (padding is never cleaned by callers)
    dag_case("dag_cfg0_ragged_translen20.npz", ragged)
    gather_case("gather_small.npz")
    print(sorted(os.listdir(HERE)))
