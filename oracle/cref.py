"""TEST INFRASTRUCTURE -- ctypes front end of oracle/dagref.c (numpy in, numpy out).

The C file is compiled by `make -C oracle` (also done by __graft_entry__.build()); if the
shared object is missing this module compiles it on first use with gcc.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libdagref.so")
_lib = None


def build(force=False):
    if force or not os.path.exists(_SO) or \
            os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_HERE, "dagref.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libdagref.so"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
    return _lib


def _p(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct))


def _f64(a):
    return np.ascontiguousarray(a, dtype=np.float64)


def _i64(a):
    return np.ascontiguousarray(a, dtype=np.int64)


def dag_loss(match, links_sq, out_len, tgt_len):
    """-> loss[B], alpha[B,T,L], beta[B,T,L] in float64."""
    match, links_sq = _f64(match), _f64(links_sq)
    out_len, tgt_len = _i64(out_len), _i64(tgt_len)
    B, T, L = match.shape
    assert links_sq.shape == (B, L, L)
    alpha = np.empty((B, T, L)); beta = np.empty((B, T, L)); loss = np.empty(B)
    d, i = ctypes.c_double, ctypes.c_int64
    lib().dagref_loss_f64(_p(match, d), _p(links_sq, d), _p(out_len, i), _p(tgt_len, i),
                          B, T, L, _p(alpha, d), _p(beta, d), _p(loss, d))
    return loss, alpha, beta


def dag_loss_grad(match, links_sq, out_len, tgt_len, g):
    """-> loss[B], grad_match[B,T,L], grad_links[B,L,L] (square) in float64."""
    match, links_sq, g = _f64(match), _f64(links_sq), _f64(g)
    out_len, tgt_len = _i64(out_len), _i64(tgt_len)
    B, T, L = match.shape
    loss, alpha, beta = dag_loss(match, links_sq, out_len, tgt_len)
    gm = np.empty((B, T, L)); gl = np.empty((B, L, L))
    d, i = ctypes.c_double, ctypes.c_int64
    lib().dagref_loss_grad_f64(_p(match, d), _p(links_sq, d), _p(out_len, i), _p(tgt_len, i),
                               _p(g, d), B, T, L, _p(alpha, d), _p(beta, d), _p(gm, d), _p(gl, d))
    return loss, gm, gl


def best_alignment(match, links_sq, out_len, tgt_len):
    """fp32 Viterbi -> path[B,L] int64, score[B] float32."""
    match = np.ascontiguousarray(match, dtype=np.float32)
    links_sq = np.ascontiguousarray(links_sq, dtype=np.float32)
    out_len, tgt_len = _i64(out_len), _i64(tgt_len)
    B, T, L = match.shape
    path = np.empty((B, L), dtype=np.int64); score = np.empty(B, dtype=np.float32)
    f, i = ctypes.c_float, ctypes.c_int64
    lib().dagref_align_f32(_p(match, f), _p(links_sq, f), _p(out_len, i), _p(tgt_len, i),
                           B, T, L, _p(path, i), _p(score, f))
    return path, score


def lsg(x, idx):
    """x [rows,V], idx [rows,S] -> sel[rows,S], lse[rows] in float64."""
    x, idx = _f64(x), _i64(idx)
    rows, V = x.shape
    S = idx.shape[1]
    sel = np.empty((rows, S)); lse = np.empty(rows)
    d, i = ctypes.c_double, ctypes.c_int64
    lib().dagref_lsg_f64(_p(x, d), _p(idx, i), rows, V, S, _p(sel, d), _p(lse, d))
    return sel, lse


def lsg_bwd(x, idx, g):
    x, idx, g = _f64(x), _i64(idx), _f64(g)
    rows, V = x.shape
    S = idx.shape[1]
    gx = np.empty((rows, V))
    d, i = ctypes.c_double, ctypes.c_int64
    lib().dagref_lsg_bwd_f64(_p(x, d), _p(idx, i), _p(g, d), rows, V, S, _p(gx, d))
    return gx
