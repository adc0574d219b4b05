"""dagx_loss_fwd_noalloc (the forward whose pipeline words live in a device array of the library) against
dagx_loss_fwd on the same inputs: two calls in a row, the second with a smaller input, every output compared
bit for bit; then the gradients computed from either set of tables."""
import ctypes

import pytest
import torch

from da_transformer_amd import _native as nat
import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _forward(entry, c, need_grad=1):
    lib = nat.lib()
    m, lk, ol, tl = c["match"], c["links"], c["out_len"], c["tgt_len"]
    B, T, L = m.shape
    tr = lk.shape[2]
    nblk = (L + 63) // 64
    # filled with a pattern first, so that cells a kernel does not write compare equal between the two runs
    hats = torch.full((2, B, T, L), 7.0, device=DEV)
    offs = torch.full((2, B, T, nblk), 7.0, dtype=torch.float64, device=DEV)
    logz = torch.full((2, B), 7.0, dtype=torch.float64, device=DEV)
    loss = torch.full((B,), 7.0, device=DEV)
    flags = torch.full((B,), 7, dtype=torch.int32, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    common = (m.data_ptr(), nat.dtype_code(m), nat.strides3(m), lk.data_ptr(), nat.dtype_code(lk), ol.data_ptr(), tl.data_ptr(),
              B, T, L, tr, hats[0].data_ptr(), hats[1].data_ptr(), offs[0].data_ptr(), offs[1].data_ptr(),
              logz.data_ptr(), loss.data_ptr(), flags.data_ptr(), need_grad)
    if entry == "noalloc":
        nat.check(lib.dagx_loss_fwd_noalloc(*common, st))
    else:
        nb = nat.workspace_bytes(nat.OP_LOSS_FWD, B, T, L, tr)
        ws = torch.zeros(max(nb, 8), dtype=torch.uint8, device=DEV)
        nat.check(lib.dagx_loss_fwd(*common, ws.data_ptr(), nb, st))
        torch.cuda.synchronize()
        assert int(ws.count_nonzero()) == 0        # the call leaves its workspace zero
    torch.cuda.synchronize()
    return hats, offs, logz, loss, flags


def _backward(c, hats, offs, logz, flags):
    lib = nat.lib()
    m, lk, ol, tl, g = c["match"], c["links"], c["out_len"], c["tgt_len"], c["grad_out"]
    B, T, L = m.shape
    tr = lk.shape[2]
    gm = torch.empty_like(m); gl = torch.empty_like(lk)
    nat.check(lib.dagx_loss_bwd(g.data_ptr(), 1, hats[0].data_ptr(), hats[1].data_ptr(), offs[0].data_ptr(), offs[1].data_ptr(),
                                logz.data_ptr(), flags.data_ptr(), m.data_ptr(), nat.dtype_code(m), nat.strides3(m),
                                lk.data_ptr(), nat.dtype_code(lk), ol.data_ptr(), tl.data_ptr(), B, T, L, tr,
                                gm.data_ptr(), gl.data_ptr(), None, 0, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return gm, gl


def test_noalloc_forward_equals_the_workspace_forward_twice_in_a_row():
    big = workloads.dag_config(1, device=DEV)                                  # B=64, L<=512, T<=64, fp16
    small = workloads.peaked_config(5, 6, 150, 40, 10.0, 5.0, device=DEV)      # smaller, ragged, pinned nodes, fp32
    for c in (big, small, big):
        got = _forward("noalloc", c)
        ref = _forward("workspace", c)
        for name, a, b in zip(("hats", "offs", "logz", "loss", "flags"), got, ref):
            assert torch.equal(a, b), name                                      # bit for bit (NaN-free by construction)
        gm, gl = _backward(c, *got[:3], got[4])
        rm, rl = _backward(c, *ref[:3], ref[4])
        assert torch.equal(gm, rm) and torch.equal(gl, rl)
        assert torch.isfinite(got[3]).all()
    # without gradients (alpha read-out) as well
    got, ref = _forward("noalloc", small, 0), _forward("workspace", small, 0)
    assert torch.equal(got[3], ref[3])


def test_noalloc_forward_allocates_nothing_and_a_cleared_workspace_serves_the_other():
    """After dagx_prepare_device (what a caller does once before capturing the entry point into a graph) the call
    changes neither the free device memory nor torch's allocator statistics; and a workspace filled with garbage,
    once cleared by dagx_loss_fwd_init_workspace, gives dagx_loss_fwd the same results."""
    lib = nat.lib()
    nat.check(lib.dagx_prepare_device())
    c = workloads.peaked_config(5, 6, 150, 40, 10.0, 5.0, device=DEV)
    m, lk, ol, tl = c["match"], c["links"], c["out_len"], c["tgt_len"]
    B, T, L = m.shape
    tr = lk.shape[2]
    nblk = (L + 63) // 64
    hats = torch.empty(2, B, T, L, device=DEV); offs = torch.empty(2, B, T, nblk, dtype=torch.float64, device=DEV)
    logz = torch.empty(2, B, dtype=torch.float64, device=DEV); loss = torch.empty(B, device=DEV)
    flags = torch.empty(B, dtype=torch.int32, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    common = (m.data_ptr(), nat.dtype_code(m), nat.strides3(m), lk.data_ptr(), nat.dtype_code(lk), ol.data_ptr(), tl.data_ptr(),
              B, T, L, tr, hats[0].data_ptr(), hats[1].data_ptr(), offs[0].data_ptr(), offs[1].data_ptr(),
              logz.data_ptr(), loss.data_ptr(), flags.data_ptr(), 1)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    stats_before = (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"])
    for _ in range(3):
        nat.check(lib.dagx_loss_fwd_noalloc(*common, st))
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.memory_stats()["allocation.all.allocated"]) == stats_before
    want = loss.clone()
    nb = nat.workspace_bytes(nat.OP_LOSS_FWD, B, T, L, tr)
    ws = torch.randint(1, 255, (max(nb, 8),), dtype=torch.uint8, device=DEV)          # garbage, as a fresh hipMalloc may hold
    nat.check(lib.dagx_loss_fwd_init_workspace(ws.data_ptr(), nb, st))
    nat.check(lib.dagx_loss_fwd(*common, ws.data_ptr(), nb, st))
    torch.cuda.synchronize()
    assert torch.equal(loss, want) and int(ws[:nb].count_nonzero()) == 0


def test_noalloc_forward_refuses_what_its_array_cannot_hold():
    lib = nat.lib()
    limit = lib.dagx_loss_fwd_noalloc_max_bytes()
    assert limit == 128 * 1024
    B, T, L = 2048, 4, 1024                      # needs far more pipeline words than the array holds
    assert nat.workspace_bytes(nat.OP_LOSS_FWD, B, T, L, L - 1) > limit
    s3 = (ctypes.c_int64 * 3)(T * L, L, 1)
    rc = lib.dagx_loss_fwd_noalloc(1, 0, s3, 1, 0, 1, 1, B, T, L, L - 1, 1, 1, 1, 1, 1, 1, 1, 1, None)
    assert rc == 2 and b"built-in scratch" in lib.dagx_last_error()
