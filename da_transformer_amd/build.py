"""Ahead-of-time build of libdagx.so (the C-ABI library with the gfx950 kernels).

    python -m da_transformer_amd.build        # or: from da_transformer_amd.build import build; build()

hipcc cross-compiles for gfx950 without a GPU.  Every source is compiled to an object file of its
own (in parallel), then linked; the library is written next to this file and loaded from there by
da_transformer_amd._native; it links against the HIP runtime only.
`python -m da_transformer_amd.build --changed` recompiles only sources newer than their objects.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
SOURCES = ["api.hip", "lsg.hip", "dag_loss.hip", "dag_align.hip", "links.hip", "glue.hip", "decode.hip", "dag_f64.hip"]
LIB = os.path.join(HERE, "libdagx.so")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-fno-fast-math", "-ffp-contract=off",
    # packed fp32 arithmetic is kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def _headers_mtime():
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    paths.append(os.path.join(ROOT, "include", "dagx.h"))
    return max(os.path.getmtime(p) for p in paths)


def build(verbose=False, extra_flags=(), only_changed=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ, exist_ok=True)
    newest_header = _headers_mtime()

    def compile_one(src):
        path, obj = os.path.join(CSRC, src), os.path.join(OBJ, src + ".o")
        if only_changed and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), newest_header):
            return obj
        cmd = [hipcc] + FLAGS + list(extra_flags) + ["-I", os.path.join(ROOT, "include"), "-I", CSRC, "-c", path, "-o", obj]
        if verbose:
            print(" ".join(cmd), file=sys.stderr)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        # the host pass does not know the (device-only) packed-fp32 feature and says so once per function: harmless
        noise = "'-packed-fp32-ops' is not a recognized feature"
        out = "\n".join(l for l in res.stdout.splitlines() if noise not in l)
        if out.strip():
            print(out, file=sys.stderr)
        if res.returncode != 0:
            raise subprocess.CalledProcessError(res.returncode, cmd)
        return obj

    with ThreadPoolExecutor(max_workers=min(len(SOURCES), os.cpu_count() or 1)) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objects)
    return LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv, only_changed="--changed" in sys.argv))
