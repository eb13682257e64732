"""ctypes binding of the C-ABI kernel library ``libxpu_graph_amd.so``.

The library is loaded on first use.  There is no CPU fallback: if the shared
object is missing the caller gets an ImportError that says how to build it.
"""
import ctypes
import os
import threading
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libxpu_graph_amd.so")

# xg_dtype / xg_act values of include/xpu_graph_amd.h
XG_F32, XG_F16, XG_BF16, XG_FP8_E4M3 = 0, 1, 2, 3
ACT_CODES = {"none": 0, "relu": 1, "gelu": 2, "silu": 3, "sigmoid": 4}
SLICE_CAT_MAX_OUTS = 32
SLICE_SUM_MAX_SLICES = 64
COMBO_SUM_MAX_JOBS = 64

_lock = threading.Lock()
_lib = None


class XgChunk(ctypes.Structure):
    _fields_ = [("src_off", ctypes.c_int32), ("dst_off", ctypes.c_int32), ("out_id", ctypes.c_int32), ("pad", ctypes.c_int32)]


class XgError(RuntimeError):
    """A C-ABI entry point refused its arguments or failed to launch."""


_SIGNATURES = {
    "xg_version": (c_int, []),
    "xg_status_string": (c_char_p, [c_int]),
    "xg_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p]),
    "xg_layer_norm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "xg_add_rms_norm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "xg_rms_norm_bwd": (c_int, [c_void_p] * 7 + [c_int64] * 6 + [c_float, c_int, c_int, c_int, c_void_p]),
    "xg_layer_norm_bwd": (c_int, [c_void_p] * 8 + [c_int64] * 6 + [c_float, c_int, c_int, c_int, c_void_p]),
    "xg_add_layer_norm": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_float, c_int, c_int, c_void_p],
    ),
    "xg_slice_cat": (
        c_int,
        [c_void_p, c_int64, c_int64, ctypes.POINTER(c_void_p), ctypes.POINTER(c_int64), c_int, c_void_p, c_int64, c_int, c_void_p],
    ),
    "xg_slice_cat_check_table": (c_int, [c_void_p, c_int64, c_int, c_int64, ctypes.POINTER(c_int64), c_int]),
    "xg_addn": (c_int, [ctypes.POINTER(c_void_p), c_int, c_void_p, c_int64, c_int, c_void_p]),
    "xg_dense_glu": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "xg_slice_sum_cat": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int32), c_int, c_int, c_void_p],
    ),
    "xg_combo_sum": (
        c_int,
        [
            ctypes.POINTER(c_void_p),
            ctypes.POINTER(c_void_p),
            ctypes.POINTER(c_int64),
            ctypes.POINTER(c_int64),
            ctypes.POINTER(c_int64),
            c_int,
            c_int,
            c_int,
            c_void_p,
        ],
    ),
    "xg_silu_mul": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "xg_silu_mul2": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "xg_dense": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "xg_dense_batched": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p] + [c_int64] * 12 + [c_int, c_int, c_int, c_int, c_void_p],
    ),
    "xg_silu_mul2_bwd": (c_int, [c_void_p] * 5 + [c_int64, c_int, c_void_p]),
    "xg_activation": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "xg_activation_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_void_p]),
    "xg_dense_glu_save": (c_int, [c_void_p] * 6 + [c_int64] * 5 + [c_int, c_void_p]),
    "xg_dense_at": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p] + [c_int64] * 6 + [c_int, c_void_p]),
    "xg_dense_fp8": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p],
    ),
    "xg_sdpa": (
        c_int,
        [
            c_void_p,
            c_void_p,
            c_void_p,
            c_void_p,
            c_int64,
            c_int64,
            c_int64,
            c_int64,
            c_int64,
            c_int64,
            ctypes.POINTER(c_int64),
            ctypes.POINTER(c_int64),
            ctypes.POINTER(c_int64),
            ctypes.POINTER(c_int64),
            c_float,
            c_int,
            c_int,
            c_void_p,
        ],
    ),
    "xg_sdpa_masked": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, ctypes.POINTER(c_int64), c_int, c_void_p]
        + [c_int64] * 6
        + [ctypes.POINTER(c_int64)] * 4
        + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_sdpa_lse": (
        c_int,
        [c_void_p] * 5 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 4 + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_sdpa_backward": (
        c_int,
        [c_void_p] * 10 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 8 + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_sdpa_decode_workspace_floats": (c_int64, [c_int64] * 6),
    "xg_sdpa_decode": (
        c_int,
        [c_void_p] * 6 + [ctypes.POINTER(c_int64), c_int, c_void_p, c_void_p] + [c_int64] * 7 + [ctypes.POINTER(c_int64)] * 4
        + [c_float, c_int, c_void_p],
    ),
    "xg_sdpa_masked_lse": (
        c_int,
        [c_void_p] * 6 + [ctypes.POINTER(c_int64), c_int, c_void_p] + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 4 + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_sdpa_backward_masked": (
        c_int,
        [c_void_p] * 7 + [ctypes.POINTER(c_int64), c_int, c_void_p] + [c_void_p] * 4 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 8
        + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_sdpa_backward_static": (
        c_int,
        [c_void_p] * 9 + [c_int64] * 6 + [ctypes.POINTER(c_int64)] * 8 + [c_float, c_int, c_int, c_void_p],
    ),
    "xg_rope": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, ctypes.POINTER(c_int64), ctypes.POINTER(c_int64), c_int64, c_int, c_int, c_void_p],
    ),
    "xg_copy_bytes": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "xg_clock_probe": (c_int, [c_void_p, c_int, c_int64, c_void_p]),
    "xg_wall_clock_khz": (c_int64, []),
}


def exported_symbols():
    """Names every build of the library must export (mirrors include/xpu_graph_amd.h)."""
    return sorted(_SIGNATURES)


def is_built():
    return os.path.exists(LIB_PATH)


def lib():
    """The loaded library; raises ImportError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: the mi355x target has no fallback path. "
                "Build it with `python -m xpu_graph_amd.build` (needs hipcc)."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError here means header and library disagree
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().xg_status_string(status).decode()
        raise XgError(f"{what} failed: {msg} (status {status})")
