"""ctypes binding of libnplm_dwconv.so (the C ABI declared in include/nplm_dwconv.h).

The library is built in-tree by ``make -C nanoplm_amd/csrc`` (or ``__graft_entry__.build()``).
There is no fallback: if the shared object is missing, every call raises.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnplm_dwconv.so")

F32 = 0
BF16 = 1
RESIDUAL = 1    # NPLM_DWCONV_RESIDUAL
GRADS_BF16 = 2  # NPLM_DWCONV_GRADS_BF16
EUNSUPPORTED = 10   # NPLM_DWCONV_EUNSUPPORTED
ESCRATCH = 11       # NPLM_DWCONV_ESCRATCH
STATIC_SCRATCH_BYTES = 16 << 20   # NPLM_DWCONV_STATIC_SCRATCH_BYTES

# every symbol include/nplm_dwconv.h declares
PUBLIC_SYMBOLS = (
    "nplm_dwconv_version",
    "nplm_dwconv_strerror",
    "nplm_dwconv_fwd",
    "nplm_dwconv_fwd_ex",
    "nplm_dwconv_bwd_workspace_bytes",
    "nplm_dwconv_bwd",
    "nplm_dwconv_bwd_ex",
    "nplm_dwconv_bwd_static",
    "nplm_dwconv_gated_fwd",
    "nplm_dwconv_gated_bwd_workspace_bytes",
    "nplm_dwconv_gated_bwd",
    "nplm_dwconv_ln_fwd",
    "nplm_dwconv_ln_bwd_workspace_bytes",
    "nplm_dwconv_ln_bwd",
    "nplm_dwconv_check_cu",
)

_lib = None


class Tuning(ctypes.Structure):
    """Mirror of ``nplm_dwconv_tuning`` (csrc/dwconv_internal.h); 0 keeps the library default."""

    _fields_ = [(n, ctypes.c_int32) for n in
                ("vec", "unroll", "tile_rows", "bw", "bt", "nbt", "xcd_remap", "maxt", "algo", "nwl", "nbuf")
                ] + [("flags", ctypes.c_uint32), ("mid_event", ctypes.c_void_p)]


def load():
    """Load the shared library once and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(the varlen depthwise conv has no non-HIP implementation)")
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, i64, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t
    lib.nplm_dwconv_version.argtypes = []
    lib.nplm_dwconv_version.restype = ctypes.c_int
    lib.nplm_dwconv_strerror.argtypes = [ctypes.c_int]
    lib.nplm_dwconv_strerror.restype = ctypes.c_char_p
    fwd_args = [vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32, vp]
    lib.nplm_dwconv_fwd.argtypes = fwd_args
    lib.nplm_dwconv_fwd.restype = ctypes.c_int
    lib.nplm_dwconv_fwd_ex.argtypes = fwd_args[:-1] + [ctypes.c_uint32, vp]
    lib.nplm_dwconv_fwd_ex.restype = ctypes.c_int
    lib.nplm_dwconv_fwd_tuned.argtypes = fwd_args + [ctypes.POINTER(Tuning)]
    lib.nplm_dwconv_fwd_tuned.restype = ctypes.c_int
    lib.nplm_dwconv_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32]
    lib.nplm_dwconv_bwd_workspace_bytes.restype = sz
    bwd_args = [vp, vp, vp, vp, vp, vp, vp, vp, sz, i64, i32, i32, i32, i32, i32, vp]
    lib.nplm_dwconv_bwd.argtypes = bwd_args
    lib.nplm_dwconv_bwd.restype = ctypes.c_int
    lib.nplm_dwconv_bwd_ex.argtypes = bwd_args[:-1] + [ctypes.c_uint32, vp]
    lib.nplm_dwconv_bwd_ex.restype = ctypes.c_int
    lib.nplm_dwconv_bwd_static.argtypes = bwd_args[:7] + bwd_args[9:-1] + [ctypes.c_uint32, vp]
    lib.nplm_dwconv_bwd_static.restype = ctypes.c_int
    lib.nplm_dwconv_gated_fwd.argtypes = fwd_args[:-1] + [ctypes.c_uint32, vp]
    lib.nplm_dwconv_gated_fwd.restype = ctypes.c_int
    lib.nplm_dwconv_ln_fwd.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, vp, vp, vp, i64, i32, i32, i32, i32, i32,
                                       ctypes.c_uint32, vp]
    lib.nplm_dwconv_ln_fwd.restype = ctypes.c_int
    lib.nplm_dwconv_ln_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32]
    lib.nplm_dwconv_ln_bwd_workspace_bytes.restype = sz
    lib.nplm_dwconv_ln_bwd.argtypes = [vp] * 13 + [sz, i64, i32, i32, i32, i32, i32, ctypes.c_uint32, vp]
    lib.nplm_dwconv_ln_bwd.restype = ctypes.c_int
    lib.nplm_dwconv_gated_bwd_workspace_bytes.argtypes = [i64, i32, i32, i32]
    lib.nplm_dwconv_gated_bwd_workspace_bytes.restype = sz
    lib.nplm_dwconv_gated_bwd.argtypes = bwd_args[:-1] + [ctypes.c_uint32, vp]
    lib.nplm_dwconv_gated_bwd.restype = ctypes.c_int
    lib.nplm_dwconv_bwd_tuned.argtypes = bwd_args + [ctypes.POINTER(Tuning)]
    lib.nplm_dwconv_bwd_tuned.restype = ctypes.c_int
    lib.nplm_dwconv_bwd_slabs.argtypes = [i64, i32, i32, i32, ctypes.POINTER(Tuning)]
    lib.nplm_dwconv_bwd_slabs.restype = i32
    lib.nplm_dwconv_exec_kernel_size.argtypes = [i32]
    lib.nplm_dwconv_exec_kernel_size.restype = i32
    lib.nplm_dwconv_debug_intervals.argtypes = [vp, i32, i64, i64, i64, i64, vp, vp]
    lib.nplm_dwconv_debug_intervals.restype = i64
    lib.nplm_dwconv_debug_copy.argtypes = [vp, vp, sz, vp]
    lib.nplm_dwconv_debug_copy.restype = ctypes.c_int
    lib.nplm_dwconv_check_cu.argtypes = [vp, i32, i64, vp]
    lib.nplm_dwconv_check_cu.restype = ctypes.c_int
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().nplm_dwconv_strerror(code).decode()


def check(code: int, what: str) -> None:
    """Raise RuntimeError carrying the library's message for a non-zero return code."""
    if code != 0:
        raise RuntimeError(f"{what} failed with code {code}: {strerror(code)}")
