"""Host side of the fused 2D neighborhood attention operator.

Mirrors the reference's Python surface (e_natten/triton.py:487-550): a
``torch.autograd.Function`` named ``Natten2d`` whose ``apply`` is exported as
``natten2d(q, k, v, kernel_size) -> out`` for ``[B, heads, H, W, d]`` tensors.
The device work is done by hand-written HIP kernels for gfx950 reached through
the C ABI of libenatten.so; the same host shims are also registered as torch
custom ops ``enatten::na2d_fwd`` / ``enatten::na2d_bwd`` (and ``na1d_*``).  There is no CPU or
eager fallback: tensors must live on the GPU and the library must be built.

Two host bindings reach the same C ABI.  ``Natten2d`` / ``Natten1d`` are Python
``autograd.Function``s over ctypes, the mirror of the reference's classes.
``natten2d`` / ``natten1d`` use the native torch binding (csrc/torch_shim.cpp,
libenatten_torch.so) when it is built: its forward and backward run no Python,
which matters because the autograd engine calls a backward on its own thread
(about a third of the host time per forward+backward on small inputs).  Without
that library they are ``Natten2d.apply`` / ``Natten1d.apply``.
"""
from __future__ import annotations

import os

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16,
           torch.float64: _lib.F64}


def _validate(q, k, v, kernel_size: int, ndim: int = 5) -> None:
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not isinstance(t, torch.Tensor):
            raise TypeError("%s must be a tensor" % name)
    if q.dim() != ndim:
        raise ValueError("expected %s tensors, got %d-D q"
                         % ("[B, heads, H, W, head_dim]" if ndim == 5 else "[B, heads, T, head_dim]",
                            q.dim()))
    if k.shape != q.shape or v.shape != q.shape:
        raise ValueError("q, k and v must have the same shape, got %s, %s, %s"
                         % (tuple(q.shape), tuple(k.shape), tuple(v.shape)))
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise ValueError("q, k and v must share a dtype")
    if q.dtype not in _DTYPES:
        raise ValueError("dtype %s is not supported (float32, bfloat16, float16, float64)" % q.dtype)
    if k.device != q.device or v.device != q.device:
        raise ValueError("q, k and v must be on the same device")
    if not isinstance(kernel_size, int) or isinstance(kernel_size, bool):
        raise TypeError("kernel_size must be an int")
    if kernel_size < 1 or kernel_size % 2 == 0:
        raise ValueError("kernel_size must be odd and >= 1, got %d" % kernel_size)
    if any(side < kernel_size for side in q.shape[2:-1]):
        raise ValueError("input of extent %s is smaller than kernel_size %d"
                         % ("x".join(str(x) for x in q.shape[2:-1]), kernel_size))
    if q.numel() == 0:
        raise ValueError("empty tensors are not supported")
    if q.shape[-1] > 1024:
        raise ValueError("head_dim %d exceeds the supported maximum of 1024" % q.shape[-1])


def _kernel_layout(t: torch.Tensor) -> torch.Tensor:
    """The kernels take any strides on the leading axes (of q, k, v, o and dO alike)
    but need unit stride on the channel axis; torch has no negative strides."""
    if t.stride(-1) != 1 and t.shape[-1] != 1:
        return t.contiguous()
    return t


def _require_gpu(t: torch.Tensor, what: str) -> None:
    # meta tensors pass: the native binding infers output shapes for them (tracing)
    if t.device.type != "cuda" and not (NATIVE_BINDING and t.device.type == "meta"):
        raise RuntimeError("%s: tensors must be on the GPU; this build has no CPU path" % what)


def _stream_of(t: torch.Tensor) -> int:
    """Raw HIP stream that torch orders work on for the tensor's device.  Called
    with that device current (the callers hold ``torch.cuda.device(t.device)``,
    which puts the previous device back when the call is over)."""
    return torch.cuda.current_stream(t.device).cuda_stream


def _check(rc: int) -> None:
    if rc != 0:
        msg = _lib.last_error()
        raise (ValueError if rc == 1 else RuntimeError)(msg)


def _fwd_impl(q, k, v, kernel_size: int, scale: float, out=None):
    """`out`: a view of the shape of q with unit stride on the channels that the kernels
    write in place (the strided sub-grid of a dilated call); None allocates the output."""
    _validate(q, k, v, kernel_size)
    _require_gpu(q, "enatten::na2d_fwd")
    lib = _lib.load()
    q, k, v = (_kernel_layout(t) for t in (q, k, v))
    B, N, H, W, D = q.shape
    with torch.cuda.device(q.device):
        # like the reference's zeros_like(Q) (e_natten/triton.py:502), the output takes
        # the memory order of q: for q sliced out of a [B, H, W, 3, heads, d] projection
        # that is [B, H, W, heads, d], which the following merge of heads needs
        o = _kernel_layout(torch.empty_like(q)) if out is None else out
        lse = torch.empty((B, N, H, W), dtype=torch.float32, device=q.device)
        _check(lib.enatten2d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                 lse.data_ptr(), B, N, H, W, D, kernel_size, _DTYPES[q.dtype],
                                 _lib.strides4(q), _lib.strides4(k), _lib.strides4(v),
                                 _lib.strides4(o), float(scale), _stream_of(q)))
    return o, lse


def _bwd_impl(q, k, v, o, lse, d_o, kernel_size: int, scale: float, out=None):
    """`out`: (dq, dk, dv) views of one layout (unit stride on the channels) that the kernels
    write in place (the strided sub-grids of a dilated call); None allocates them."""
    _validate(q, k, v, kernel_size)
    _require_gpu(q, "enatten::na2d_bwd")
    if d_o.shape != q.shape or o.shape != q.shape:
        raise ValueError("o and d_o must have the shape of q")
    if d_o.dtype != q.dtype or o.dtype != q.dtype:
        raise ValueError("o and d_o must have the dtype of q")
    lib = _lib.load()
    q, k, v, o, d_o = (_kernel_layout(t) for t in (q, k, v, o, d_o))
    lse = lse.contiguous()
    B, N, H, W, D = q.shape
    with torch.cuda.device(q.device):
        if out is None:
            dq = torch.empty((B, N, H, W, D), dtype=q.dtype, device=q.device)
            dk, dv = torch.empty_like(dq), torch.empty_like(dq)
        else:
            dq, dk, dv = out
            assert dq.stride() == dk.stride() == dv.stride() and dq.stride(-1) == 1
        ws = torch.empty(lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, kernel_size,
                                                            _DTYPES[q.dtype]),
                         dtype=torch.uint8, device=q.device)
        _check(lib.enatten2d_bwd_into(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                      d_o.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                      dv.data_ptr(), ws.data_ptr(), B, N, H, W, D, kernel_size,
                                      _DTYPES[q.dtype], _lib.strides4(q), _lib.strides4(k),
                                      _lib.strides4(v), _lib.strides4(o), _lib.strides4(d_o),
                                      None if out is None else _lib.strides4(dq),
                                      float(scale), _stream_of(q)))
    return dq, dk, dv


def _fwd1d_impl(q, k, v, kernel_size: int, scale: float, out=None):
    _validate(q, k, v, kernel_size, 4)
    _require_gpu(q, "enatten::na1d_fwd")
    lib = _lib.load()
    q, k, v = (_kernel_layout(t) for t in (q, k, v))
    B, N, T, D = q.shape
    with torch.cuda.device(q.device):
        o = _kernel_layout(torch.empty_like(q)) if out is None else out
        lse = torch.empty((B, N, T), dtype=torch.float32, device=q.device)
        _check(lib.enatten1d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                 lse.data_ptr(), B, N, T, D, kernel_size, _DTYPES[q.dtype],
                                 _lib.strides3(q), _lib.strides3(k), _lib.strides3(v),
                                 _lib.strides3(o), float(scale), _stream_of(q)))
    return o, lse


def _bwd1d_impl(q, k, v, o, lse, d_o, kernel_size: int, scale: float, out=None):
    _validate(q, k, v, kernel_size, 4)
    _require_gpu(q, "enatten::na1d_bwd")
    if d_o.shape != q.shape or o.shape != q.shape:
        raise ValueError("o and d_o must have the shape of q")
    if d_o.dtype != q.dtype or o.dtype != q.dtype:
        raise ValueError("o and d_o must have the dtype of q")
    lib = _lib.load()
    q, k, v, o, d_o = (_kernel_layout(t) for t in (q, k, v, o, d_o))
    lse = lse.contiguous()
    B, N, T, D = q.shape
    with torch.cuda.device(q.device):
        if out is None:
            dq = torch.empty((B, N, T, D), dtype=q.dtype, device=q.device)
            dk, dv = torch.empty_like(dq), torch.empty_like(dq)
        else:
            dq, dk, dv = out
            assert dq.stride() == dk.stride() == dv.stride() and dq.stride(-1) == 1
        ws = torch.empty(lib.enatten1d_bwd_workspace_bytes(B, N, T), dtype=torch.uint8,
                         device=q.device)
        _check(lib.enatten1d_bwd_into(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                      d_o.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                                      dv.data_ptr(), ws.data_ptr(), B, N, T, D, kernel_size,
                                      _DTYPES[q.dtype], _lib.strides3(q), _lib.strides3(k),
                                      _lib.strides3(v), _lib.strides3(o), _lib.strides3(d_o),
                                      None if out is None else _lib.strides3(dq),
                                      float(scale), _stream_of(q)))
    return dq, dk, dv


def _load_native_binding() -> bool:
    """Load libenatten_torch.so, which registers the enatten:: operators from C++.
    It needs libenatten.so beside it; with either file missing the operators are
    registered from Python below (and fail at the first call if libenatten.so is
    missing)."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libenatten_torch.so")
    if os.environ.get("ENATTEN_PYTHON_BINDING") == "1":
        return False
    if not (os.path.exists(path) and os.path.exists(_lib.LIB_PATH)):
        return False
    try:
        _lib.load()
    except ImportError:  # stale or broken build: every call will say so; importing must
        return False     # still work, or `python -m e_natten_amd.build` could not run
    try:
        torch.ops.load_library(path)
    except OSError as e:  # built against another torch: keep working through Python
        import warnings
        warnings.warn("e_natten_amd: %s does not load (%s); using the Python binding. Rebuild it "
                      "with `python -m e_natten_amd.build`." % (path, e), RuntimeWarning)
        return False
    return True


NATIVE_BINDING = _load_native_binding()

if not NATIVE_BINDING:
    # torch custom ops: thin shims over the C ABI
    _torch_lib = torch.library.Library("enatten", "DEF")
    _torch_lib.define("na2d_fwd(Tensor q, Tensor k, Tensor v, int kernel_size, float scale) "
                      "-> (Tensor, Tensor)")
    _torch_lib.define("na2d_bwd(Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, Tensor d_o, "
                      "int kernel_size, float scale) -> (Tensor, Tensor, Tensor)")
    _torch_lib.impl("na2d_fwd", _fwd_impl, "CompositeExplicitAutograd")
    _torch_lib.impl("na2d_bwd", _bwd_impl, "CompositeExplicitAutograd")
    _torch_lib.define("na1d_fwd(Tensor q, Tensor k, Tensor v, int kernel_size, float scale) "
                      "-> (Tensor, Tensor)")
    _torch_lib.define("na1d_bwd(Tensor q, Tensor k, Tensor v, Tensor o, Tensor lse, Tensor d_o, "
                      "int kernel_size, float scale) -> (Tensor, Tensor, Tensor)")
    _torch_lib.impl("na1d_fwd", _fwd1d_impl, "CompositeExplicitAutograd")
    _torch_lib.impl("na1d_bwd", _bwd1d_impl, "CompositeExplicitAutograd")


class Natten2d(torch.autograd.Function):
    """2D neighborhood attention, ``[B, heads, H, W, d]`` in and out.

    Same contract as the reference Function (e_natten/triton.py:487-548):
    ``forward(ctx, Q, K, V, kernel_size=7)``; ``backward`` returns
    ``(dQ, dK, dV, None)``.  The logits carry no softmax scale, as in the
    reference; the optional fifth argument ``scale`` multiplies them.  The
    forward also keeps each query's log-sum-exp so the backward can recompute
    the probabilities without a second softmax reduction.
    """

    @staticmethod
    def forward(ctx, Q, K, V, kernel_size=7, scale=1.0):
        o, lse = _fwd_impl(Q, K, V, kernel_size, scale)
        ctx.save_for_backward(Q, K, V, o, lse)
        ctx.kernel_size = kernel_size
        ctx.scale = scale
        return o

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        Q, K, V, o, lse = ctx.saved_tensors
        dQ, dK, dV = _bwd_impl(Q, K, V, o, lse, grad_output, ctx.kernel_size, ctx.scale)
        return dQ, dK, dV, None, None


class Natten2dDilated(torch.autograd.Function):
    """Dilated 2D neighborhood attention: query (x, y) attends the kernel_size^2 keys
    that are `dilation` apart around it (NATTEN's dilated neighborhood; the reference
    has no dilation and always passes 1 to its comparator, test.py:17).  Pixels with
    equal (x mod dilation, y mod dilation) only ever see each other, and inside such
    a sub-grid the rule is the plain one, so the operator is the undilated kernels run
    on the dilation^2 strided sub-grids of q, k, v (the C ABI takes strides), each
    writing its own pixels of the output in place (the C ABI takes the strides of o)."""

    @staticmethod
    def forward(ctx, Q, K, V, kernel_size, scale, dilation):
        o = torch.empty(Q.shape, dtype=Q.dtype, device=Q.device)
        lses = []
        for i in range(dilation):
            for j in range(dilation):
                sub = (slice(None), slice(None), slice(i, None, dilation), slice(j, None, dilation))
                _, lse_s = _fwd_impl(Q[sub], K[sub], V[sub], kernel_size, scale, out=o[sub])
                lses.append(lse_s)
        ctx.save_for_backward(Q, K, V, o, *lses)
        ctx.args = (kernel_size, scale, dilation)
        return o

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        Q, K, V, o, *lses = ctx.saved_tensors
        kernel_size, scale, dilation = ctx.args
        dQ, dK, dV = (torch.empty(Q.shape, dtype=Q.dtype, device=Q.device) for _ in range(3))
        for i in range(dilation):
            for j in range(dilation):
                sub = (slice(None), slice(None), slice(i, None, dilation), slice(j, None, dilation))
                _bwd_impl(Q[sub], K[sub], V[sub], o[sub], lses[i * dilation + j], grad_output[sub],
                          kernel_size, scale, out=(dQ[sub], dK[sub], dV[sub]))
        return dQ, dK, dV, None, None, None


def _pair(x, what, kind):
    """An int / bool or a pair of them -> a pair."""
    if isinstance(x, (tuple, list)):
        if len(x) != 2:
            raise ValueError("%s must have one entry per image axis" % what)
        x = tuple(x)
    else:
        x = (x, x)
    for e in x:
        if kind is int and (not isinstance(e, int) or isinstance(e, bool)):
            raise TypeError("%s must be an int or a pair of ints" % what)
        if kind is bool and not isinstance(e, (bool, int)):
            raise TypeError("%s must be a bool or a pair of bools" % what)
    return x if kind is int else (bool(x[0]), bool(x[1]))


def _validate_window(q, k, v, kernel, causal) -> None:
    _validate(q, k, v, 1)
    for L, ks, c, axis in zip(q.shape[2:4], kernel, causal, ("rows", "columns")):
        if ks < 1 or (not c and ks % 2 == 0):
            raise ValueError("kernel_size along %s must be >= 1, and odd unless that axis is "
                             "causal, got %d" % (axis, ks))
        if L < ks:
            raise ValueError("input has %d %s, fewer than kernel_size %d" % (L, axis, ks))


def _validate_rpb(q, rpb, kernel, causal) -> None:
    if not isinstance(rpb, torch.Tensor):
        raise TypeError("rpb must be a tensor")
    want = (q.shape[1], 2 * kernel[0] - 1, 2 * kernel[1] - 1)
    if tuple(rpb.shape) != want:
        raise ValueError("rpb must have shape [heads, 2*kh-1, 2*kw-1] = %s, got %s"
                         % (list(want), list(rpb.shape)))
    if rpb.dtype != q.dtype or rpb.device != q.device:
        raise ValueError("rpb must have the dtype and device of q")
    if any(causal):
        raise ValueError("a relative position bias goes with centred axes only")


def _window_fwd(q, k, v, rpb, kernel, causal, scale: float):
    _validate_window(q, k, v, kernel, causal)
    if rpb is not None:
        _validate_rpb(q, rpb, kernel, causal)
        rpb = rpb.contiguous()
    _require_gpu(q, "natten2d")
    if q.device.type != "cuda":
        raise RuntimeError("natten2d: rectangular and causal windows need tensors on the GPU")
    lib = _lib.load()
    q, k, v = (_kernel_layout(t) for t in (q, k, v))
    B, N, H, W, D = q.shape
    with torch.cuda.device(q.device):
        o = _kernel_layout(torch.empty_like(q))
        lse = torch.empty((B, N, H, W), dtype=torch.float32, device=q.device)
        _check(lib.enatten2d_fwd_window(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), rpb.data_ptr() if rpb is not None else None,
            o.data_ptr(), lse.data_ptr(), B, N, H, W, D,
            kernel[0], kernel[1], int(causal[0]), int(causal[1]), _DTYPES[q.dtype],
            _lib.strides4(q), _lib.strides4(k), _lib.strides4(v), _lib.strides4(o), float(scale),
            _stream_of(q)))
    return o, lse


def _window_bwd(q, k, v, rpb, o, lse, d_o, kernel, causal, scale: float):
    lib = _lib.load()
    q, k, v, o, d_o = (_kernel_layout(t) for t in (q, k, v, o, d_o))
    B, N, H, W, D = q.shape
    with torch.cuda.device(q.device):
        dq = torch.empty((B, N, H, W, D), dtype=q.dtype, device=q.device)
        dk, dv = torch.empty_like(dq), torch.empty_like(dq)
        d_rpb = None
        if rpb is not None:
            rpb = rpb.contiguous()
            d_rpb = torch.empty(rpb.shape, dtype=torch.float32, device=q.device)
        ws = torch.empty(lib.enatten2d_bwd_window_workspace_bytes(B, N, H, W, kernel[0], kernel[1],
                                                                  int(rpb is not None)),
                         dtype=torch.uint8, device=q.device)
        _check(lib.enatten2d_bwd_window(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), rpb.data_ptr() if rpb is not None else None,
            o.data_ptr(), d_o.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(),
            dv.data_ptr(), d_rpb.data_ptr() if rpb is not None else None, ws.data_ptr(),
            B, N, H, W, D, kernel[0],
            kernel[1], int(causal[0]), int(causal[1]), _DTYPES[q.dtype], _lib.strides4(q),
            _lib.strides4(k), _lib.strides4(v), _lib.strides4(o), _lib.strides4(d_o), float(scale),
            _stream_of(q)))
    return dq, dk, dv, (d_rpb.to(q.dtype) if rpb is not None else None)


class Natten2dWindow(torch.autograd.Function):
    """2D neighborhood attention with a rectangular and / or causal window (NATTEN's
    definitions; the reference has one odd kernel_size and no causal mode):
    ``kernel = (rows, columns)``, ``causal = (rows, columns)``.  On a causal axis a query
    attends the last k positions up to and including its own.  ``rpb`` is None or a
    relative position bias ``[heads, 2*rows-1, 2*columns-1]`` that is added to the scaled
    logits (entry key - query + kernel - 1 per axis) and gets a gradient.  Served by the
    general kernels through ``enatten2d_fwd_window`` / ``enatten2d_bwd_window``."""

    @staticmethod
    def forward(ctx, Q, K, V, rpb, kernel, causal, scale):
        o, lse = _window_fwd(Q, K, V, rpb, kernel, causal, scale)
        ctx.save_for_backward(Q, K, V, o, lse, *(() if rpb is None else (rpb,)))
        ctx.args = (kernel, causal, scale)
        return o

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        Q, K, V, o, lse, *rest = ctx.saved_tensors
        dQ, dK, dV, d_rpb = _window_bwd(Q, K, V, rest[0] if rest else None, o, lse, grad_output,
                                        *ctx.args)
        return dQ, dK, dV, d_rpb, None, None, None


def _window_call(q, k, v, kernel, causal, scale, dilation, rpb=None):
    """Natten2dWindow on the dilation^2 strided sub-grids (see Natten2dDilated)."""
    if dilation == 1:
        return Natten2dWindow.apply(q, k, v, rpb, kernel, causal, float(scale))
    if not isinstance(dilation, int) or isinstance(dilation, bool) or dilation < 1:
        raise ValueError("dilation must be a positive int")
    _validate_window(q, k, v, kernel, causal)
    for L, ks in zip(q.shape[2:4], kernel):
        if L > 1 and L < ks * dilation:
            raise ValueError("input of extent %d is smaller than kernel_size * dilation = %d"
                             % (L, ks * dilation))
    o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    for i in range(dilation if q.shape[2] > 1 else 1):
        for j in range(dilation):
            sub = (slice(None), slice(None),
                   slice(i, None, dilation) if q.shape[2] > 1 else slice(None),
                   slice(j, None, dilation))
            o[sub] = Natten2dWindow.apply(q[sub], k[sub], v[sub], rpb, kernel, causal, float(scale))
    return o


def natten2d(q, k, v, kernel_size=7, scale=1.0, dilation=1, is_causal=False, rpb=None):
    """``natten2d(q, k, v, kernel_size) -> out`` on ``[B, heads, H, W, d]`` tensors,
    differentiable in q, k and v: the reference's entry point
    (e_natten/triton.py:550, e_natten/__init__.py:1), positional like it.
    ``dilation`` > 1 spaces every neighborhood's keys that far apart (needs image sides
    of at least kernel_size * dilation).  Beyond the reference, as in NATTEN:
    ``kernel_size`` may be a pair (rows, columns), and ``is_causal`` (a bool or a pair)
    makes an axis causal: a query then attends the last kernel_size positions up to and
    including its own; ``rpb`` is a relative position bias ``[heads, 2*kh-1, 2*kw-1]`` added
    to the scaled logits (differentiable too)."""
    if isinstance(kernel_size, (tuple, list)) or is_causal is not False or rpb is not None:
        kernel, causal = _pair(kernel_size, "kernel_size", int), _pair(is_causal, "is_causal", bool)
        if kernel[0] != kernel[1] or any(causal) or rpb is not None:
            return _window_call(q, k, v, kernel, causal, scale, dilation, rpb)
        kernel_size = kernel[0]
    if dilation != 1:
        if not isinstance(dilation, int) or isinstance(dilation, bool) or dilation < 1:
            raise ValueError("dilation must be a positive int")
        _validate(q, k, v, kernel_size)
        _require_gpu(q, "natten2d")
        if min(q.shape[2], q.shape[3]) < kernel_size * dilation:
            raise ValueError("input of extent %dx%d is smaller than kernel_size * dilation = %d"
                             % (q.shape[2], q.shape[3], kernel_size * dilation))
        return Natten2dDilated.apply(q, k, v, kernel_size, float(scale), dilation)
    if not NATIVE_BINDING:
        return Natten2d.apply(q, k, v, kernel_size, scale)
    # the native operator checks shapes, dtypes, devices and the kernel size itself and raises
    # the same error classes (csrc/torch_shim.cpp: validate); only the argument's Python type
    # is checked here, once, so that a float or a bool is not silently converted
    if type(kernel_size) is not int:
        raise TypeError("kernel_size must be an int")
    return torch.ops.enatten.natten2d(q, k, v, kernel_size, float(scale))


class Natten1d(torch.autograd.Function):
    """1D neighborhood attention, ``[B, heads, T, d]`` in and out; same contract
    as the reference Function (e_natten/triton.py:425-483)."""

    @staticmethod
    def forward(ctx, q, k, v, kernel_size=7, scale=1.0):
        o, lse = _fwd1d_impl(q, k, v, kernel_size, scale)
        ctx.save_for_backward(q, k, v, o, lse)
        ctx.kernel_size = kernel_size
        ctx.scale = scale
        return o

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        q, k, v, o, lse = ctx.saved_tensors
        dQ, dK, dV = _bwd1d_impl(q, k, v, o, lse, grad_output, ctx.kernel_size, ctx.scale)
        return dQ, dK, dV, None, None


class Natten1dDilated(torch.autograd.Function):
    """Dilated 1D neighborhood attention: the undilated kernels on the `dilation`
    strided sub-sequences (see Natten2dDilated)."""

    @staticmethod
    def forward(ctx, q, k, v, kernel_size, scale, dilation):
        o = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        lses = []
        for i in range(dilation):
            sub = (slice(None), slice(None), slice(i, None, dilation))
            _, lse_s = _fwd1d_impl(q[sub], k[sub], v[sub], kernel_size, scale, out=o[sub])
            lses.append(lse_s)
        ctx.save_for_backward(q, k, v, o, *lses)
        ctx.args = (kernel_size, scale, dilation)
        return o

    @staticmethod
    @torch.autograd.function.once_differentiable
    def backward(ctx, grad_output):
        q, k, v, o, *lses = ctx.saved_tensors
        kernel_size, scale, dilation = ctx.args
        dQ, dK, dV = (torch.empty(q.shape, dtype=q.dtype, device=q.device) for _ in range(3))
        for i in range(dilation):
            sub = (slice(None), slice(None), slice(i, None, dilation))
            _bwd1d_impl(q[sub], k[sub], v[sub], o[sub], lses[i], grad_output[sub], kernel_size,
                        scale, out=(dQ[sub], dK[sub], dV[sub]))
        return dQ, dK, dV, None, None, None


def natten1d(q, k, v, kernel_size=7, scale=1.0, dilation=1, is_causal=False, rpb=None):
    """``natten1d(q, k, v, kernel_size) -> out`` on ``[B, heads, T, d]`` tensors
    (e_natten/triton.py:485, e_natten/__init__.py:1).  ``dilation`` as in natten2d;
    ``is_causal=True`` (not in the reference) is sliding-window causal attention: query t
    attends keys max(t - kernel_size + 1, 0) .. t; ``rpb`` is a relative position bias
    ``[heads, 2*kernel_size-1]``."""
    if is_causal or rpb is not None:
        _validate(q, k, v, 1, 4)
        if not isinstance(kernel_size, int) or isinstance(kernel_size, bool):
            raise TypeError("kernel_size must be an int")
        if rpb is not None and (not isinstance(rpb, torch.Tensor) or rpb.dim() != 2):
            raise ValueError("rpb must be a [heads, 2*kernel_size-1] tensor")
        o = _window_call(q.unsqueeze(2), k.unsqueeze(2), v.unsqueeze(2), (1, kernel_size),
                         (False, bool(is_causal)), scale, dilation,
                         None if rpb is None else rpb.unsqueeze(1))
        return o.squeeze(2)
    if dilation != 1:
        if not isinstance(dilation, int) or isinstance(dilation, bool) or dilation < 1:
            raise ValueError("dilation must be a positive int")
        _validate(q, k, v, kernel_size, 4)
        _require_gpu(q, "natten1d")
        if q.shape[2] < kernel_size * dilation:
            raise ValueError("sequence of %d positions is shorter than kernel_size * dilation = %d"
                             % (q.shape[2], kernel_size * dilation))
        return Natten1dDilated.apply(q, k, v, kernel_size, float(scale), dilation)
    if not NATIVE_BINDING:
        return Natten1d.apply(q, k, v, kernel_size, scale)
    if type(kernel_size) is not int:   # everything else is checked by the native operator
        raise TypeError("kernel_size must be an int")
    return torch.ops.enatten.natten1d(q, k, v, kernel_size, float(scale))


def kernel_path(head_dim: int, kernel_size: int, dtype: torch.dtype) -> str:
    """Which kernel family serves a configuration: 'mfma', 'simt' or 'none'."""
    code = _lib.load().enatten2d_kernel_path(head_dim, kernel_size, _DTYPES.get(dtype, -1))
    return {_lib.PATH_MFMA: "mfma", _lib.PATH_SIMT: "simt"}.get(code, "none")
