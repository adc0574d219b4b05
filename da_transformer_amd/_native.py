"""ctypes binding of libdagx.so (the C ABI declared in include/dagx.h).

There is no fallback: if the library is missing or a call fails, a RuntimeError is raised.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdagx.so")

F32, F16, BF16 = 0, 1, 2
OP_LOSS_FWD, OP_LOSS_BWD, OP_BEST_ALIGNMENT, OP_VITERBI_DECODE, OP_BEST_ALIGNMENT_F64 = 0, 1, 2, 3, 4

_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_lib = None

_vp, _i, _i64, _sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t
_Strides = ctypes.c_int64 * 3

EXPORTS = {
    "dagx_version": (ctypes.c_char_p, []),
    "dagx_last_error": (ctypes.c_char_p, []),
    "dagx_force_log_domain": (_i, [_i]),
    "dagx_loss_float64_first": (_i, [_i]),
    "dagx_workspace_bytes": (_sz, [_i, _i, _i, _i, _i]),
    "dagx_lsg_fwd": (_i, [_vp, _i, _i, _i, _i64, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dagx_lsg_bwd": (_i, [_vp, _i, _i, _i, _i64, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dagx_lsg_fwd_argmax": (_i, [_vp, _i, _i, _i, _i64, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dagx_loss_fwd": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                           _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _sz, _vp]),
    "dagx_loss_fwd_init_workspace": (_i, [_vp, _sz, _vp]),
    "dagx_prepare_device": (_i, []),
    "dagx_loss_fwd_noalloc_max_bytes": (_sz, []),
    "dagx_loss_fwd_noalloc": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                                   _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp]),
    "dagx_loss_bwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i,
                           _vp, _vp, _vp, _sz, _vp]),
    "dagx_best_alignment": (_i, [_vp, _i, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "dagx_links_fwd": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dagx_links_bwd": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "dagx_force_emit": (_i, [_vp, _i, _vp, _vp, _i, _i, _i, _i, _vp, _vp]),
    "dagx_viterbi_decode": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i64,
                                 _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "dagx_lookahead_decode": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _i, ctypes.c_float, _i, _i64, _vp, _vp, _vp, _vp]),
    "dagx_loss_f64_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp, _i, _vp]),
    "dagx_loss_f64_bwd": (_i, [_vp, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "dagx_best_alignment_f64": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _sz, _vp]),
    "dagx_lsg_f64_fwd": (_i, [_vp, _i, _i, _i64, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dagx_lsg_f64_bwd": (_i, [_vp, _i, _i, _i64, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "dagx_glat_glance": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_float, _i, _i, _i, _i,
                              _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
}


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m da_transformer_amd.build` "
                "(the DAG operators have no non-HIP fallback)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in EXPORTS.items():
            fn = getattr(handle, name)
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def version():
    return lib().dagx_version().decode()


def dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise RuntimeError(f"dagx: unsupported dtype {t.dtype} (float32, float16 and bfloat16 are)") from None


def strides3(t):
    return _Strides(*t.stride())


def ptr(t):
    return None if t is None else t.data_ptr()


def stream_of(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def check(rc):
    if rc != 0:
        raise RuntimeError("dagx: " + lib().dagx_last_error().decode())


def workspace_bytes(op, B, T, L, translen):
    return int(lib().dagx_workspace_bytes(op, B, T, L, translen))
