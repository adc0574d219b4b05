"""Ahead-of-time build of libdagx.so (the C-ABI library with the gfx950 kernels).

    python -m da_transformer_amd.build        # or: from da_transformer_amd.build import build; build()

hipcc cross-compiles for gfx950 without a GPU.  The library is written next to this file and
loaded from there by da_transformer_amd._native; it links against the HIP runtime only.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
SOURCES = ["api.hip", "lsg.hip", "dag_loss.hip", "dag_align.hip", "links.hip", "glue.hip", "decode.hip"]
LIB = os.path.join(HERE, "libdagx.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-fno-fast-math", "-ffp-contract=off",
    # packed fp32 arithmetic is kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build(verbose=False, extra_flags=()):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + list(extra_flags) + [
        "-I", os.path.join(ROOT, "include"), "-I", CSRC,
        "-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES]
    if verbose:
        print(" ".join(cmd), file=sys.stderr)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
