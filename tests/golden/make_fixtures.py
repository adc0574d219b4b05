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


if __name__ == "__main__":
    dag_case("dag_cfg0.npz", workloads.dag_config(0))
    ragged = workloads.dag_config(0, translen=20)
    ragged["out_len"] = torch.tensor([64, 50, 33, 17]); ragged["tgt_len"] = torch.tensor([16, 9, 16, 2])
    # rows beyond L_b keep stale finite values on purpose (padding is never cleaned by callers)
    dag_case("dag_cfg0_ragged_translen20.npz", ragged)
    gather_case("gather_small.npz")
    print(sorted(os.listdir(HERE)))
