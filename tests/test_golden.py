"""Committed golden vectors (tests/golden/*.npz, written by make_golden.py from the
fp64 oracle): every CPU statement reproduces them, and so do the HIP kernels."""
import glob
import os

import numpy as np
import pytest
import torch

from _util import FP32_MAX_ABS, O, ROOT, ensure_built
from oracle import na1d_oracle as O1
from oracle import na2d_c

FILES = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "*.npz")))


def _load(path):
    z = np.load(path, allow_pickle=False)
    t = {k: torch.from_numpy(z[k]) for k in ("q", "k", "v", "d_o", "o", "lse", "dq", "dk", "dv")}
    return t, int(z["kernel_size"]), float(z["scale"])


def test_fixtures_exist():
    assert len(FILES) >= 4


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_cpu_statements_reproduce_golden(path):
    t, ks, scale = _load(path)
    if t["q"].dim() == 5:
        got = O.natten2d_gather_grads(t["q"], t["k"], t["v"], t["d_o"], ks, scale)
        oc, lc = na2d_c.forward(t["q"], t["k"], t["v"], ks, scale)
        gc = na2d_c.backward(t["q"], t["k"], t["v"], t["d_o"], ks, scale)
    else:
        got = O1.natten1d_explicit(t["q"], t["k"], t["v"], t["d_o"], ks, scale)
        oc, lc = na2d_c.forward_1d(t["q"], t["k"], t["v"], ks, scale)
        gc = na2d_c.backward_1d(t["q"], t["k"], t["v"], t["d_o"], ks, scale)
    for name, x in zip(("o", "lse", "dq", "dk", "dv"), got):
        assert O.max_abs_err(x, t[name]) < 2e-6, name  # fixtures are stored in float32
    for name, x in zip(("o", "lse", "dq", "dk", "dv"), (oc, lc) + tuple(gc)):
        assert O.max_abs_err(x, t[name]) < 2e-5, name


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f) for f in FILES])
def test_gpu_reproduces_golden(path):
    ensure_built()
    from e_natten_amd import Natten1d, Natten2d
    t, ks, scale = _load(path)
    fn = Natten2d if t["q"].dim() == 5 else Natten1d
    q, k, v = (t[n].cuda().requires_grad_(True) for n in ("q", "k", "v"))
    o = fn.apply(q, k, v, ks, scale)
    o.backward(t["d_o"].cuda())
    for name, x in (("o", o), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        assert O.max_abs_err(x.detach().cpu(), t[name]) < FP32_MAX_ABS, name
