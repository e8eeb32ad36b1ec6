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
    from e_natten_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from e_natten_amd import build
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


def run_gpu(q, k, v, d_o, ks, scale=1.0):
    """Forward + backward of the HIP operator through autograd on cuda:0."""
    from e_natten_amd import Natten2d
    dev = torch.device("cuda:0")
    qg, kg, vg = (t.to(dev).requires_grad_(True) for t in (q, k, v))
    o = Natten2d.apply(qg, kg, vg, ks, scale)
    o.backward(d_o.to(dev))
    torch.cuda.synchronize()
    return tuple(t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad))


def assert_close(got, ref, dtype, what):
    names = ("O", "dQ", "dK", "dV")
    for name, x, r in zip(names, got, ref):
        assert torch.isfinite(x.float()).all(), "%s: %s has non-finite values" % (what, name)
        if dtype == torch.float32:
            err = O.max_abs_err(x, r)
            print("   %s %s max-abs err %.3e" % (what, name, err), flush=True)
            assert err <= FP32_MAX_ABS, "%s: %s max-abs err %.3e > %.0e" % (what, name, err, FP32_MAX_ABS)
        else:
            err = O.rel_err(x, r)
            print("   %s %s rel err %.3e" % (what, name, err), flush=True)
            assert err <= BF16_REL, "%s: %s rel err %.3e > %.0e" % (what, name, err, BF16_REL)
