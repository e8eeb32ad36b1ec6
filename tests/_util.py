"""Shared helpers of the parity tests: seeded inputs per benchmark
configuration and comparison against the CPU oracle."""
from __future__ import annotations

import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import na2d_c, na2d_oracle as O  # noqa: E402

# tolerances of the operator's contract
FP32_MAX_ABS = 1e-4   # float32: max |x - ref| on O, dQ, dK, dV
BF16_REL = 2e-2       # bfloat16 / float16: max |x - ref| / max |ref|


def ensure_built():
    """Load the HIP library; build it only if no built library is present."""
    from e_natten_amd import _lib, build
    if not (os.path.exists(_lib.LIB_PATH) and os.path.exists(build.TORCH_LIB)):
        build.build()
    return _lib.load()


def make_inputs(shape, dtype, seed=0, q_scale=1.0, k_scale=1.0):
    """q, k, v, dO ~ N(0,1) drawn on the CPU in float32 from `seed`, scaled,
    then rounded to `dtype` (the oracle sees exactly these rounded values)."""
    g = torch.Generator().manual_seed(seed)
    q, k, v, d_o = (torch.randn(shape, generator=g, dtype=torch.float32) for _ in range(4))
    q, k = q * q_scale, k * k_scale
    return tuple(t.to(dtype) for t in (q, k, v, d_o))


def oracle_all(q, k, v, d_o, ks, scale=1.0, small=False):
    """(O, LSE, dQ, dK, dV) on the CPU.  `small` uses the fp64 torch gather
    oracle, otherwise the C oracle (double accumulation, float32 storage)."""
    if small:
        return O.natten2d_explicit(q, k, v, d_o, ks, scale)
    o, lse = na2d_c.forward(q, k, v, ks, scale)
    dq, dk, dv = na2d_c.backward(q, k, v, d_o, ks, scale)
    return o, lse, dq, dk, dv


def _poison_free_blocks(shape, dtype, dev):
    """Leave NaN-filled blocks of the operator's output sizes as the only free
    blocks of torch's caching allocator, so that an output element the kernels
    fail to write shows up as NaN instead of a stale result of an earlier case."""
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    junk = [torch.full(shape, float("nan"), dtype=dtype, device=dev) for _ in range(4)]
    junk += [torch.full(shape[:-1], float("nan"), dtype=torch.float32, device=dev) for _ in range(2)]
    torch.cuda.synchronize()
    del junk


def run_gpu(q, k, v, d_o, ks, scale=1.0, binding="native"):
    """Forward + backward of the HIP operator through autograd on cuda:0, through
    `natten2d` (the native torch binding where it is built) or, with
    binding="python", through the Python autograd.Function."""
    from e_natten_amd import Natten2d, natten2d
    dev = torch.device("cuda:0")
    qg, kg, vg = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    _poison_free_blocks(tuple(q.shape), q.dtype, dev)
    o = (natten2d if binding == "native" else Natten2d.apply)(qg, kg, vg, ks, scale)
    o.backward(d_o.to(dev))
    torch.cuda.synchronize()
    return tuple(t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad))


def run_capi(q, k, v, d_o, ks, scale=1.0):
    """Forward + backward straight through the C ABI into buffers that hold NaN
    everywhere beforehand: returns (O, LSE, dQ, dK, dV) on the CPU."""
    from e_natten_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    code = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}[q.dtype]
    qd, kd, vd, gd = (t.to(dev).contiguous() for t in (q, k, v, d_o))
    B, N, H, W, D = q.shape
    o, dq, dk, dv = (torch.full_like(qd, float("nan")) for _ in range(4))
    lse = torch.full((B, N, H, W), float("nan"), dtype=torch.float32, device=dev)
    ws = torch.full((lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, ks, code) // 4 + 1,), float("nan"),
                    dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.enatten2d_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(),
                           lse.data_ptr(), B, N, H, W, D, ks, code, None, None, None, None,
                           float(scale), st)
    assert rc == 0, _lib.last_error()
    rc = lib.enatten2d_bwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(),
                           gd.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                           dv.data_ptr(), ws.data_ptr(), B, N, H, W, D, ks, code, None, None,
                           None, None, None, float(scale), st)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return tuple(t.cpu() for t in (o, lse, dq, dk, dv))


def assert_close(got, ref, dtype, what):
    """float32: max |x - ref| <= 1e-4.  bfloat16 / float16: max |x - ref| <= 2e-2 *
    max |ref| per tensor, and beside it the elementwise form of the same bound,
    allclose(rtol=2e-2, atol=2e-2 * max |ref|), which the first implies; both are
    printed and asserted."""
    names = ("O", "dQ", "dK", "dV")
    for name, x, r in zip(names, got, ref):
        assert torch.isfinite(x.float()).all(), "%s: %s has non-finite values" % (what, name)
        if dtype == torch.float32:
            err = O.max_abs_err(x, r)
            print("   %s %s max-abs err %.3e" % (what, name, err), flush=True)
            assert err <= FP32_MAX_ABS, "%s: %s max-abs err %.3e > %.0e" % (what, name, err, FP32_MAX_ABS)
        else:
            err = O.rel_err(x, r)
            xd, rd = x.double(), r.double()
            atol = BF16_REL * rd.abs().max().item()
            elementwise = torch.allclose(xd, rd, rtol=BF16_REL, atol=atol)
            worst = ((xd - rd).abs() / (atol + BF16_REL * rd.abs())).max().item()
            print("   %s %s rel err %.3e; allclose(rtol=2e-2, atol=2e-2*max|ref|) %s, worst "
                  "element at %.3f of its bound" % (what, name, err, elementwise, worst), flush=True)
            assert err <= BF16_REL, "%s: %s rel err %.3e > %.0e" % (what, name, err, BF16_REL)
            assert elementwise, "%s: %s fails allclose(rtol=2e-2, atol=2e-2*max|ref|)" % (what, name)
