"""ctypes access to the C oracle (oracle/na2d_ref.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libna2d_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/na2d_ref.c with gcc into libna2d_oracle.so."""
    args = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(args, check=True, capture_output=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        fp = ctypes.POINTER(ctypes.c_float)
        L.na2d_win_start.restype = ctypes.c_int
        L.na2d_win_start.argtypes = [ctypes.c_int] * 3
        L.na2d_inv_range.restype = None
        L.na2d_inv_range.argtypes = [ctypes.c_int] * 3 + [ctypes.POINTER(ctypes.c_int)] * 2
        L.na2d_max_threads.restype = ctypes.c_int
        L.na2d_fwd_f32.restype = None
        L.na2d_fwd_f32.argtypes = [fp] * 5 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int]
        L.na2d_bwd_f32.restype = None
        L.na2d_bwd_f32.argtypes = [fp] * 7 + [ctypes.c_int] * 5 + [ctypes.c_float, ctypes.c_int]
        L.na2d_fwd_rect_f32.restype = None
        L.na2d_fwd_rect_f32.argtypes = [fp] * 5 + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_int]
        L.na2d_bwd_rect_f32.restype = None
        L.na2d_bwd_rect_f32.argtypes = [fp] * 7 + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_int]
        _lib = L
    return _lib


def _p(t: torch.Tensor):
    return ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_float))


def win_start(i: int, L: int, k: int) -> int:
    return lib().na2d_win_start(i, L, k)


def inv_range(i: int, L: int, k: int):
    lo, hi = ctypes.c_int(), ctypes.c_int()
    lib().na2d_inv_range(i, L, k, ctypes.byref(lo), ctypes.byref(hi))
    return lo.value, hi.value


def _prep(*ts):
    return [t.detach().to("cpu", torch.float32).contiguous() for t in ts]


def forward(q, k, v, kernel_size: int, scale: float = 1.0, nthreads: int = 0):
    """(O, LSE) as float32 CPU tensors; inputs of any float dtype are widened."""
    q, k, v = _prep(q, k, v)
    B, N, H, W, D = q.shape
    o = torch.empty_like(q)
    lse = torch.empty(B, N, H, W, dtype=torch.float32)
    lib().na2d_fwd_f32(_p(q), _p(k), _p(v), _p(o), _p(lse), B * N, H, W, D,
                       kernel_size, scale, nthreads)
    return o, lse


def backward(q, k, v, d_o, kernel_size: int, scale: float = 1.0, nthreads: int = 0):
    """(dQ, dK, dV) as float32 CPU tensors."""
    q, k, v, d_o = _prep(q, k, v, d_o)
    B, N, H, W, D = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    lib().na2d_bwd_f32(_p(q), _p(k), _p(v), _p(d_o), _p(dq), _p(dk), _p(dv),
                       B * N, H, W, D, kernel_size, scale, nthreads)
    return dq, dk, dv


def forward_1d(q, k, v, kernel_size: int, scale: float = 1.0, nthreads: int = 0):
    """1D operator on [B, heads, T, d]: (O, LSE) through the 1 x k rectangular window."""
    q, k, v = _prep(q, k, v)
    B, N, T, D = q.shape
    o = torch.empty_like(q)
    lse = torch.empty(B, N, T, dtype=torch.float32)
    lib().na2d_fwd_rect_f32(_p(q), _p(k), _p(v), _p(o), _p(lse), B * N, 1, T, D, 1,
                            kernel_size, scale, nthreads)
    return o, lse


def backward_1d(q, k, v, d_o, kernel_size: int, scale: float = 1.0, nthreads: int = 0):
    q, k, v, d_o = _prep(q, k, v, d_o)
    B, N, T, D = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    lib().na2d_bwd_rect_f32(_p(q), _p(k), _p(v), _p(d_o), _p(dq), _p(dk), _p(dv),
                            B * N, 1, T, D, 1, kernel_size, scale, nthreads)
    return dq, dk, dv
