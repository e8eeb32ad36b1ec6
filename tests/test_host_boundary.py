"""Host side and C-ABI surface, without a GPU: the library loads, exports every
symbol the header declares, validates arguments before touching the device, and
the Python entry points mirror the reference's signature."""
import ctypes
import inspect
import os
import re

import pytest
import torch

from _util import ROOT, ensure_built


@pytest.fixture(scope="module")
def lib():
    return ensure_built()


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "enatten.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(enatten\w*)\s*\(", text)))


def test_library_exports_every_declared_symbol(lib):
    from e_natten_amd import _lib
    names = _declared_functions()
    assert "enatten2d_fwd" in names and "enatten2d_bwd" in names
    for n in names:
        assert hasattr(lib, n), "libenatten.so does not export %s" % n
    assert sorted(_lib.SIGNATURES) == names
    assert lib.enatten_abi_version() == _lib.ABI_VERSION == 5


def test_c_abi_validates_before_launch(lib):
    from e_natten_amd import _lib
    f = lambda ks, H=8, W=8, D=16, dt=0, q=1: lib.enatten2d_fwd(
        q, 1, 1, 1, None, 1, 1, H, W, D, ks, dt, None, None, None, None, 1.0, None)
    assert f(4) == 1 and "odd" in _lib.last_error()
    assert f(-1) == 1
    assert f(9) == 1 and "smaller" in _lib.last_error()
    assert f(3, dt=7) == 1 and "dtype" in _lib.last_error()
    assert f(3, D=0) == 1
    assert f(3, q=None) == 1 and "NULL" in _lib.last_error()
    assert lib.enatten2d_bwd(1, 1, 1, 1, 1, None, 1, 1, 1, 1, 1, 1, 8, 8, 16, 3, 0,
                             None, None, None, None, None, 1.0, None) == 1
    # negative strides are refused for every strided tensor, the output included
    neg = (ctypes.c_int64 * 4)(1024, 512, -128, 16)
    assert lib.enatten2d_fwd(1, 1, 1, 1, None, 1, 1, 8, 8, 16, 3, 0, None, None, None, neg,
                             1.0, None) == 1 and "negative stride for o" in _lib.last_error()
    # more than 2^40 elements: refused as unsupported, before any pointer is looked at
    assert lib.enatten2d_fwd(None, 1, 1, 1, None, 1 << 12, 1 << 12, 1 << 12, 1 << 12, 1024, 3, 0,
                             None, None, None, None, 1.0, None) == 2
    assert lib.enatten2d_bwd_workspace_bytes(2, 3, 4, 5, 64, 3, 1) == 2 * 3 * 4 * 5 * 8
    assert lib.enatten2d_bwd_workspace_bytes(0, 3, 4, 5, 64, 3, 1) == 0
    # the float32 matrix-core backward keeps P and dS of every window position
    assert lib.enatten2d_bwd_workspace_bytes(2, 3, 8, 8, 128, 5, 0) == 2 * 3 * 8 * 8 * 2 * 25 * 4
    assert lib.enatten2d_bwd_workspace_bytes(2, 3, 16, 16, 128, 9, 0) == 2 * 3 * 16 * 16 * 8


def test_kernel_path_query(lib):
    from e_natten_amd import kernel_path
    assert kernel_path(128, 5, torch.float32) == "mfma"    # float32 matrix-core kernels
    assert kernel_path(128, 9, torch.float32) == "simt"
    # every kernel size of the matrix-core kernels at head_dim 128, the largest windows included
    assert all(kernel_path(128, ks, torch.bfloat16) == "mfma" for ks in (3, 5, 7, 9, 11, 13))
    assert kernel_path(128, 13, torch.float16) == "mfma" and kernel_path(128, 15, torch.bfloat16) == "simt"
    # multiples of 8 below the built head dims run on the next one's kernels (not 64 with k 11, 13)
    assert all(kernel_path(d, 5, torch.bfloat16) == "mfma" for d in (8, 16, 24, 40, 48, 56, 72, 96, 120))
    assert kernel_path(48, 13, torch.bfloat16) == "simt" and kernel_path(96, 13, torch.float16) == "mfma"
    assert kernel_path(20, 5, torch.bfloat16) == "simt" and kernel_path(256, 5, torch.bfloat16) == "simt"
    assert kernel_path(2, 3, torch.float32) == "simt"
    assert kernel_path(128, 4, torch.bfloat16) == "none"
    assert kernel_path(4096, 3, torch.bfloat16) == "none"
    assert kernel_path(128, 5, torch.float64) == "simt"    # float64: kernels of their own, not matrix-core
    assert kernel_path(128, 5, torch.int32) == "none"
    prev = lib.enatten_set_path(1)
    assert kernel_path(128, 5, torch.bfloat16) == "simt"
    lib.enatten_set_path(prev)


def test_native_torch_binding_registers_operators():
    # libenatten_torch.so (csrc/torch_shim.cpp) loads without a GPU and registers the
    # operators from C++; its checks raise the same error classes as the Python side
    from e_natten_amd import ops
    assert ops.NATIVE_BINDING, "libenatten_torch.so is not built or failed to load"
    for name in ("na2d_fwd", "na2d_bwd", "na1d_fwd", "na1d_bwd", "natten2d", "natten1d"):
        assert hasattr(torch.ops.enatten, name)
    q = torch.randn(1, 1, 8, 8, 16)
    with pytest.raises(ValueError, match="odd"):
        torch.ops.enatten.natten2d(q, q, q, 4, 1.0)
    with pytest.raises(ValueError, match="smaller"):
        torch.ops.enatten.natten2d(q, q, q, 9, 1.0)
    with pytest.raises(ValueError, match="same shape"):
        torch.ops.enatten.na2d_fwd(q, q[:, :, :4], q, 3, 1.0)
    with pytest.raises(ValueError, match="dtype"):
        torch.ops.enatten.natten2d(q.int(), q.int(), q.int(), 3, 1.0)
    with pytest.raises(RuntimeError, match="no CPU path"):
        torch.ops.enatten.natten2d(q, q, q, 3, 1.0)
    with pytest.raises(RuntimeError, match="no CPU path"):
        torch.ops.enatten.natten1d(q[0], q[0], q[0], 3, 1.0)


def test_python_binding_can_be_forced():
    # ENATTEN_PYTHON_BINDING=1 keeps the native binding out: the operators are then
    # registered from Python and natten2d is the Python Function's apply
    import subprocess
    import sys
    code = ("import torch, e_natten_amd\n"
            "from e_natten_amd import ops\n"
            "assert not ops.NATIVE_BINDING\n"
            "assert hasattr(torch.ops.enatten, 'na2d_fwd')\n"
            "q = torch.randn(1, 1, 8, 8, 16)\n"
            "try:\n"
            "    e_natten_amd.natten2d(q, q, q, 3)\n"
            "except RuntimeError as e:\n"
            "    assert 'no CPU path' in str(e)\n"
            "else:\n"
            "    raise SystemExit('CPU tensors were accepted')\n")
    env = dict(os.environ, ENATTEN_PYTHON_BINDING="1", PYTHONPATH=ROOT)
    r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]


def test_python_surface_mirrors_reference():
    import e_natten_amd
    from e_natten_amd import Natten2d, natten2d
    # e_natten/triton.py:489: forward(ctx, Q, K, V, kernel_size=7)
    params = list(inspect.signature(Natten2d.forward).parameters.values())
    assert [p.name for p in params[:5]] == ["ctx", "Q", "K", "V", "kernel_size"]
    assert params[4].default == 7
    assert natten2d == Natten2d.apply or callable(natten2d)
    assert "natten2d" in e_natten_amd.__all__


def test_1d_surface_and_validation(lib):
    from e_natten_amd import Natten1d, _lib, natten1d
    params = list(inspect.signature(Natten1d.forward).parameters.values())
    assert [p.name for p in params[:5]] == ["ctx", "q", "k", "v", "kernel_size"]
    assert params[4].default == 7  # e_natten/triton.py:427
    q = torch.randn(1, 2, 8, 16)
    for bad in (4, 0, 9):
        with pytest.raises(ValueError):
            natten1d(q, q, q, bad)
    with pytest.raises(ValueError):
        natten1d(q[0], q[0], q[0], 3)
    with pytest.raises(RuntimeError, match="no CPU path"):
        natten1d(q, q, q, 3)
    f = lambda ks, T=8: lib.enatten1d_fwd(1, 1, 1, 1, None, 1, 1, T, 16, ks, 0, None, None,
                                          None, None, 1.0, None)
    assert f(4) == 1 and "odd" in _lib.last_error()
    assert f(9) == 1 and "smaller" in _lib.last_error()
    assert lib.enatten1d_bwd_workspace_bytes(2, 3, 10) == 2 * 3 * 10 * 16  # two doubles per position for float64 tensors
    # The size limit is on B * heads * T * D elements, not on a T x T image: long
    # sequences pass it and fail on the NULL pointer that follows (nothing is launched).
    for B, N, T, D in ((8, 8, 16384, 128), (1, 8, 131072, 64), (1, 1, 1 << 22, 64)):
        rc = lib.enatten1d_fwd(None, 1, 1, 1, None, B, N, T, D, 7, 1, None, None, None, None,
                               1.0, None)
        assert rc == 1 and "q is NULL" in _lib.last_error(), (B, N, T, D, _lib.last_error())
    assert lib.enatten1d_fwd(None, 1, 1, 1, None, 1 << 10, 1 << 10, 1 << 20, 1024, 7, 1, None,
                             None, None, None, 1.0, None) == 2


def test_python_validation_without_gpu():
    from e_natten_amd import natten2d
    q = torch.randn(1, 1, 8, 8, 16)
    for bad in (4, 0, 9):
        with pytest.raises(ValueError):
            natten2d(q, q, q, bad)
    with pytest.raises(ValueError):
        natten2d(q[0], q[0], q[0], 3)
    with pytest.raises(ValueError):
        natten2d(q, q[:, :, :4], q, 3)
    with pytest.raises(ValueError):
        natten2d(q.int(), q.int(), q.int(), 3)
    with pytest.raises(TypeError):
        natten2d(q, q, q, 3.0)
    # valid arguments on CPU tensors: there is no CPU path, so this must fail loudly
    with pytest.raises(RuntimeError, match="no CPU path"):
        natten2d(q, q, q, 3)


def test_product_package_does_not_import_oracle():
    pkg = os.path.join(ROOT, "e_natten_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower() or f == "never", (f, "mentions the oracle")


def test_meta_tensors_give_shapes_without_a_gpu():
    # shape inference for tracing: the native operators accept meta tensors, validate them
    # like real ones and return outputs (and gradients) of the right shape and dtype
    from e_natten_amd import natten1d, natten2d, ops
    if not ops.NATIVE_BINDING:
        pytest.skip("native torch binding not built")
    q = torch.empty(2, 3, 16, 12, 64, device="meta", dtype=torch.bfloat16, requires_grad=True)
    o = natten2d(q, q, q, 5)
    assert o.shape == q.shape and o.dtype == q.dtype and o.device.type == "meta"
    (g,) = torch.autograd.grad(o, q, torch.empty_like(o))
    assert g.shape == q.shape
    o2, lse = torch.ops.enatten.na2d_fwd(q.detach(), q.detach(), q.detach(), 5, 1.0)
    assert lse.shape == q.shape[:-1] and lse.dtype == torch.float32
    s = torch.empty(2, 3, 100, 32, device="meta", dtype=torch.float16)
    assert natten1d(s, s, s, 7).shape == s.shape
    with pytest.raises(ValueError):
        natten2d(q, q, q, 4)


def test_window_entry_points_validate(lib):
    from e_natten_amd import _lib, natten1d, natten2d
    f = lambda kh, kw, ch=0, cw=0, H=8, W=8, q=1, rpb=None: lib.enatten2d_fwd_window(
        q, 1, 1, rpb, 1, None, 1, 1, H, W, 16, kh, kw, ch, cw, 0, None, None, None, None, 1.0, None)
    assert f(3, 4) == 1 and "odd unless that axis is causal" in _lib.last_error()
    assert f(9, 3) == 1 and "fewer than kernel_h" in _lib.last_error()
    assert f(3, 0, 0, 1) == 1
    assert f(3, 4, 0, 1, q=None) == 1 and "q is NULL" in _lib.last_error()   # even is fine when causal
    assert f(4, 4) == 1 and "odd" in _lib.last_error()   # square non-causal: the plain entry point's rule
    assert lib.enatten2d_bwd_window_workspace_bytes(2, 3, 4, 5, 3, 7, 0) == 2 * 3 * 4 * 5 * 16
    assert lib.enatten2d_bwd_window_workspace_bytes(2, 3, 4, 5, 3, 7, 1) == 2 * 3 * 4 * 5 * (16 + 21 * 4)
    assert f(3, 5, 0, 1, rpb=1) == 1 and "centred axes only" in _lib.last_error()
    assert lib.enatten2d_bwd_window(1, 1, 1, None, 1, 1, None, 1, 1, 1, None, None, 1, 1, 8, 8, 16, 3, 5,
                                    0, 0, 0, None, None, None, None, None, 1.0, None) == 1
    assert "workspace is NULL" in _lib.last_error()
    assert lib.enatten2d_bwd_window(1, 1, 1, 1, 1, 1, None, 1, 1, 1, None, 1, 1, 1, 8, 8, 16, 3, 5,
                                    0, 0, 0, None, None, None, None, None, 1.0, None) == 1
    assert "rpb and d_rpb come together" in _lib.last_error()
    q = torch.randn(1, 2, 8, 8, 16)
    with pytest.raises(ValueError, match="odd unless"):
        natten2d(q, q, q, (3, 4))
    with pytest.raises(ValueError, match="fewer than"):
        natten2d(q, q, q, (9, 3))
    with pytest.raises(ValueError, match="one entry per image axis"):
        natten2d(q, q, q, (3, 3, 3))
    with pytest.raises(TypeError):
        natten2d(q, q, q, (3, 3.0))
    with pytest.raises(RuntimeError, match="no CPU path"):
        natten2d(q, q, q, (3, 5))
    with pytest.raises(RuntimeError, match="no CPU path"):
        natten1d(q[0], q[0], q[0], 4, is_causal=True)
    with pytest.raises(ValueError):
        natten1d(q[0], q[0], q[0], 9, is_causal=True)
    with pytest.raises(ValueError, match="rpb must have shape"):
        natten2d(q, q, q, 3, rpb=torch.zeros(2, 5, 7))
    with pytest.raises(ValueError, match="centred axes only"):
        natten2d(q, q, q, 3, is_causal=(True, False), rpb=torch.zeros(2, 5, 5))
    with pytest.raises(RuntimeError, match="no CPU path"):
        natten2d(q, q, q, 3, rpb=torch.zeros(2, 5, 5))
