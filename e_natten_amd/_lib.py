"""ctypes binding of libenatten.so (the C ABI declared in include/enatten.h)."""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libenatten.so")

ABI_VERSION = 5  # ENATTEN_ABI_VERSION of include/enatten.h
F32, BF16, F16, F64 = 0, 1, 2, 3
STATIC_BWD_MAX_QUERIES = 1 << 20
PATH_NONE, PATH_SIMT, PATH_MFMA, PATH_MFMA_FUSED, PATH_MFMA_SPLIT = 0, 1, 2, 3, 4
PATH_MFMA_SPLIT_QUEUE = 5

_lock = threading.Lock()
_lib = None

_vp = ctypes.c_void_p
_i = ctypes.c_int
_sp = ctypes.POINTER(ctypes.c_int64)

# name -> (restype, argtypes); kept in step with include/enatten.h
SIGNATURES = {
    "enatten_abi_version": (_i, []),
    "enatten_last_error": (ctypes.c_char_p, []),
    "enatten2d_kernel_path": (_i, [_i, _i, _i]),
    "enatten_set_path": (_i, [_i]),
    "enatten2d_fwd": (_i, [_vp] * 5 + [_i] * 7 + [_sp] * 4 + [ctypes.c_float, _vp]),
    "enatten2d_bwd_workspace_bytes": (ctypes.c_size_t, [_i] * 7),
    "enatten2d_bwd": (_i, [_vp] * 10 + [_i] * 7 + [_sp] * 5 + [ctypes.c_float, _vp]),
    "enatten2d_bwd_into": (_i, [_vp] * 10 + [_i] * 7 + [_sp] * 6 + [ctypes.c_float, _vp]),
    "enatten2d_bwd_static": (_i, [_vp] * 9 + [_i] * 7 + [_sp] * 5 + [ctypes.c_float, _vp]),
    "enatten2d_fwd_window": (_i, [_vp] * 6 + [_i] * 10 + [_sp] * 4 + [ctypes.c_float, _vp]),
    "enatten2d_bwd_window_workspace_bytes": (ctypes.c_size_t, [_i] * 7),
    "enatten2d_bwd_window": (_i, [_vp] * 12 + [_i] * 10 + [_sp] * 5 + [ctypes.c_float, _vp]),
    "enatten1d_fwd": (_i, [_vp] * 5 + [_i] * 6 + [_sp] * 4 + [ctypes.c_float, _vp]),
    "enatten1d_bwd_workspace_bytes": (ctypes.c_size_t, [_i] * 3),
    "enatten1d_bwd": (_i, [_vp] * 10 + [_i] * 6 + [_sp] * 5 + [ctypes.c_float, _vp]),
    "enatten1d_bwd_into": (_i, [_vp] * 10 + [_i] * 6 + [_sp] * 6 + [ctypes.c_float, _vp]),
    "enatten_profile_enable": (_i, [_i]),
    "enatten_profile_read": (_i, [_i, ctypes.POINTER(_i), ctypes.POINTER(ctypes.c_double)]),
    "enatten_profile_read_overhead": (_i, [_i, ctypes.POINTER(ctypes.c_double)]),
    "enatten_profile_kernel_name": (ctypes.c_char_p, [_i]),
}


def load() -> ctypes.CDLL:
    """Load libenatten.so.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise ImportError(
                    "%s is missing: build it with `python -m e_natten_amd.build` "
                    "(needs hipcc; cross-compiles for gfx950 without a GPU)" % LIB_PATH)
            lib = ctypes.CDLL(LIB_PATH)
            stale = "%s is stale (%%s): rebuild it with `python -m e_natten_amd.build`" % LIB_PATH
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(lib, name, None)
                if fn is None:
                    raise ImportError(stale % ("it does not export %s" % name))
                fn.restype, fn.argtypes = res, args
            if lib.enatten_abi_version() != ABI_VERSION:
                raise ImportError(stale % "unexpected ABI version")
            _lib = lib
    return _lib


def last_error() -> str:
    return load().enatten_last_error().decode()


def strides3(t) -> ctypes.Array:
    """Element strides of the (batch, head, position) axes as int64_t[3]."""
    return (ctypes.c_int64 * 3)(*t.stride()[:3])


def strides4(t) -> ctypes.Array:
    """Element strides of the (batch, head, row, column) axes as int64_t[4]."""
    return (ctypes.c_int64 * 4)(*t.stride()[:4])
