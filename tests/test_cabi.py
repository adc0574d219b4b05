"""The C-ABI library loads and exports every symbol include/dagx.h declares (no compute calls)."""
import ctypes
import os
import re

import pytest
import torch

from conftest import ROOT
from da_transformer_amd import _native


def _declared():
    text = open(os.path.join(ROOT, "include", "dagx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dagx_[a-z_0-9]+)\s*\(", text)))


def test_header_declares_the_entry_points():
    names = _declared()
    for want in ("dagx_version", "dagx_last_error", "dagx_force_log_domain", "dagx_workspace_bytes", "dagx_lsg_fwd", "dagx_lsg_bwd",
                 "dagx_loss_fwd", "dagx_loss_bwd", "dagx_best_alignment", "dagx_links_fwd", "dagx_links_bwd",
                 "dagx_force_emit", "dagx_glat_glance", "dagx_viterbi_decode", "dagx_lookahead_decode"):
        assert want in names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_native.LIB_PATH), "build libdagx.so first: python -m da_transformer_amd.build"
    handle = ctypes.CDLL(_native.LIB_PATH)
    for name in _declared():
        assert hasattr(handle, name), name
    assert set(_declared()) == set(_native.EXPORTS), "python binding and header disagree"
    assert b"gfx950" in ctypes.cast(handle.dagx_version, ctypes.CFUNCTYPE(ctypes.c_char_p))()


def test_argument_errors_are_reported_without_a_gpu():
    lib = _native.lib()
    s3 = (ctypes.c_int64 * 3)(1, 1, 1)
    rc = lib.dagx_lsg_fwd(None, 0, 1, 1, 10, 1, None, s3, None, s3, None, None)
    assert rc == 1 and b"null pointer" in lib.dagx_last_error()
    rc = lib.dagx_loss_fwd(1, 7, s3, 1, 0, 1, 1, 1, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, 0, None)
    assert rc == 1 and b"dtype" in lib.dagx_last_error()
    rc = lib.dagx_best_alignment(1, 0, s3, 1, 0, 1, 1, 1, 2, 9000, 1, 1, None, 0, None)
    assert rc == 2 and b"8192" in lib.dagx_last_error()
    # alignment: score table + pipeline words + flags, plus an int32 trace when back-pointers do not fit LDS
    assert lib.dagx_workspace_bytes(_native.OP_BEST_ALIGNMENT, 16, 256, 1024, 1023) == \
        4 * (16 * 256 * 1024 + 16 + 16 * 10 + 16 + 4) + 16 * 256 * 1024 + 16 * 256 * 1024 * 4
    # score table, ticket/progress words, flags, alignment slack, one source-block byte per cell
    assert lib.dagx_workspace_bytes(_native.OP_BEST_ALIGNMENT, 64, 64, 512, 511) == \
        4 * (64 * 64 * 512 + 16 + 64 * 4 + 64 + 4) + 64 * 64 * 512
    # loss forward: the pipeline's ticket/progress words, two counters per sample, then the fast kernel's two read-outs per sample
    assert lib.dagx_workspace_bytes(_native.OP_LOSS_FWD, 64, 64, 512, 511) == 4 * (16 + 2 * 64 * 2 + 2 * 64) + 8 * 2 * 64
    assert lib.dagx_workspace_bytes(_native.OP_LOSS_FWD, 4, 16, 2048, 2047) == 0     # log-domain kernel only
    assert lib.dagx_workspace_bytes(_native.OP_LOSS_BWD, 64, 64, 512, 511) == 0
    rc = lib.dagx_loss_fwd(1, 0, s3, 1, 0, 1, 1, 1, 2, 2, 1, 1, 1, 1, 1, 1, 1, 1, 1, None, 0, None)
    assert rc == 3 and b"workspace" in lib.dagx_last_error()


def test_argument_errors_of_the_wider_entry_points_without_a_gpu():
    lib = _native.lib()
    s3 = (ctypes.c_int64 * 3)(1, 1, 1)
    rc = lib.dagx_links_fwd(1, 0, 1, 1, 2, 8, 5, 7, 1, 1, None)
    assert rc == 2 and b"heads" in lib.dagx_last_error()
    rc = lib.dagx_force_emit(1, 0, s3, 1, 2, 0, 4, 0, 1, None)
    assert rc == 1 and b"bad sizes" in lib.dagx_last_error()
    rc = lib.dagx_force_emit(None, 0, s3, 1, 2, 3, 4, 0, 1, None)
    assert rc == 1 and b"null pointer" in lib.dagx_last_error()
    rc = lib.dagx_glat_glance(1, 1, 1, 1, None, 1, 1, None, 0.5, 2, 3, 4, 2, 1, 1, 1, 1, 1, 1, None)
    assert rc == 1 and b"keep_prob_in" in lib.dagx_last_error()           # the mix stage alone needs a keep probability
    rc = lib.dagx_glat_glance(1, 1, 1, 1, None, 1, 1, None, 0.5, 2, 3, 4, 4, 1, 1, 1, 1, 1, 1, None)
    assert rc == 1 and b"stages" in lib.dagx_last_error()
    rc = lib.dagx_viterbi_decode(1, 0, 1, 1, 1, 2, 2048, 2047, 64, 1, 1, 1, 1, 1, 1, 1, None, 0, None)
    assert rc == 2 and b"1024" in lib.dagx_last_error()
    rc = lib.dagx_viterbi_decode(1, 0, 1, 1, 1, 2, 512, 511, 128, 1, 1, 1, 1, 1, 1, 1, None, 0, None)
    assert rc == 3 and b"workspace" in lib.dagx_last_error()
    # decoding: score table of max_length + 1 rows, pipeline words, flags, slack, source blocks, three match rows
    assert lib.dagx_workspace_bytes(_native.OP_VITERBI_DECODE, 64, 128, 512, 511) == \
        4 * (64 * 129 * 512 + 16 + 64 * 4 + 64 + 4 + 64 * 3 * 512) + 64 * 129 * 512
    rc = lib.dagx_lookahead_decode(1, 0, 1, 1, 1, 2, 5000, 100, 1.0, 0, 1, 1, 1, 1, None)
    assert rc == 2 and b"4096" in lib.dagx_last_error()
    rc = lib.dagx_lookahead_decode(1, 3, 1, 1, 1, 2, 50, 10, 1.0, 0, 1, 1, 1, 1, None)
    assert rc == 1 and b"dtype" in lib.dagx_last_error()


def test_operators_refuse_cpu_tensors():
    import da_transformer_amd as d
    with pytest.raises(RuntimeError):
        d.dag_loss(torch.zeros(1, 2, 2), torch.zeros(1, 2, 1), torch.tensor([2]), torch.tensor([2]))
    with pytest.raises(RuntimeError):
        d.dag_logsoftmax_gather_inplace(torch.zeros(1, 2, 5), torch.zeros(1, 2, 1, dtype=torch.long))


def test_torch_versions_match_the_oracle_on_cpu():
    """The package's public torch_* functions (selectable torch path) agree with the oracle."""
    import da_transformer_amd as d
    from oracle import torch_native as tn
    from helpers import random_problem
    match, links, ol, tl = random_problem(42, 3, 20, 7, dtype=torch.float32, drop=0.1)
    assert torch.equal(d.torch_dag_loss(match, links, ol, tl), tn.torch_dag_loss(match, links, ol, tl))
    assert torch.equal(d.torch_dag_best_alignment(match, links, ol, tl),
                       tn.torch_dag_best_alignment(match, links, ol, tl))
    sh = d.extract_valid_links(links)
    assert torch.equal(sh, tn.extract_valid_links(links))
    assert torch.equal(d.restore_valid_links(sh), tn.restore_valid_links(sh))
    x = torch.randn(2, 3, 11); idx = torch.randint(0, 11, (2, 3, 4))
    assert torch.equal(d.torch_dag_logsoftmax_gather_inplace(x, idx)[1],
                       tn.torch_dag_logsoftmax_gather_inplace(x, idx)[1])
    force = torch.full((3, 20), -1, dtype=torch.long); force[:, 5] = 2
    assert torch.equal(d.force_alignment(match, force), tn.force_alignment(match, force))


def test_golden_fixtures_agree_with_the_torch_oracle():
    import numpy as np
    from oracle import torch_native as tn
    for name in ("dag_cfg0.npz", "dag_cfg0_ragged_translen20.npz"):
        z = np.load(os.path.join(ROOT, "tests", "golden", name))
        match = torch.from_numpy(z["match"]).double().requires_grad_()
        links = torch.from_numpy(z["links"]).double().requires_grad_()
        ol, tl = torch.from_numpy(z["out_len"]), torch.from_numpy(z["tgt_len"])
        loss = tn.torch_dag_loss(match, tn.restore_valid_links(links), ol, tl)
        assert np.allclose(loss.detach().numpy(), z["loss"], rtol=1e-10)
        gm, gl = torch.autograd.grad((loss * torch.from_numpy(z["grad_out"]).double()).sum(), [match, links])
        assert np.allclose(gm.numpy(), z["grad_match"], rtol=1e-5, atol=1e-9)
        assert np.allclose(gl.numpy(), z["grad_links"], rtol=1e-5, atol=1e-9)


def test_a_missing_library_is_an_error_not_a_fallback(monkeypatch):
    """Without libdagx.so every operator raises: nothing falls back to PyTorch or to the CPU."""
    import da_transformer_amd as d
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", os.path.join(ROOT, "da_transformer_amd", "no_such_libdagx.so"))
    with pytest.raises(RuntimeError, match="missing"):
        _native.lib()
    with pytest.raises(RuntimeError):
        d.dag_loss(torch.zeros(1, 2, 2), torch.zeros(1, 2, 1), torch.tensor([2]), torch.tensor([2]))
    with pytest.raises(RuntimeError):
        d.dag_viterbi_decode(torch.zeros(1, 4, 3), (torch.zeros(1, 4), torch.zeros(1, 4, dtype=torch.long)), torch.tensor([4]), 2.0, 1.0, True, 1)


def test_header_is_valid_c_and_cpp_and_a_c_program_links_against_the_library(tmp_path):
    """The boundary is plain C: the header compiles as C99 and as C++11 on its own, and a C program that names
    every declared entry point links against libdagx.so (nothing is called: no GPU here)."""
    import shutil
    import subprocess
    header_dir = os.path.join(ROOT, "include")
    gcc, gxx = shutil.which("gcc"), shutil.which("g++")
    if not gcc or not gxx:
        pytest.skip("no host compiler")
    subprocess.run([gcc, "-fsyntax-only", "-x", "c", "-std=c99", "-Wall", "-Wextra", "-Werror", os.path.join(header_dir, "dagx.h")], check=True)
    subprocess.run([gxx, "-fsyntax-only", "-x", "c++", "-std=c++11", "-Wall", "-Werror", os.path.join(header_dir, "dagx.h")], check=True)
    src = tmp_path / "link_all.c"
    names = _declared()
    src.write_text('#include "dagx.h"\n#include <stdio.h>\nint main(void) {\n  const void *entry[] = {'
                   + ", ".join("(const void *)" + n for n in names)
                   + '};\n  printf("%s: %d entry points\\n", dagx_version(), (int)(sizeof entry / sizeof entry[0]));\n  return entry[0] == 0;\n}\n')
    exe = tmp_path / "link_all"
    libdir = os.path.dirname(_native.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wno-pedantic", "-I", header_dir, str(src), "-o", str(exe), "-L", libdir, "-l:libdagx.so",
                    "-Wl,-rpath," + libdir], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert "gfx950" in out and f"{len(names)} entry points" in out
