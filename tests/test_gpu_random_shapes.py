"""Seeded random shapes through the C ABI against the CPU oracle: every kernel family
(16-bit matrix-core, float32 matrix-core, 1D matrix-core, general), both backward paths,
ragged and tile-aligned images, batch * heads from 1 to hundreds; rectangular and causal
windows and the relative position bias against the dense-mask oracle."""
import random

import pytest
import torch

from _util import BF16_REL, FP32_MAX_ABS, O, ensure_built, make_inputs, oracle_all, run_capi
from oracle import na1d_oracle as O1

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def lib():
    assert torch.cuda.is_available()
    return ensure_built()


def _cases_2d(n, seed):
    rnd = random.Random(seed)
    out = []
    for it in range(n):
        dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        D = rnd.choice([32, 64, 64, 128, 128, 48] if dt != torch.float32 else [32, 64, 128, 128, 24])
        ks = rnd.choice([3, 5, 5, 7, 7, 9, 11, 13] if dt != torch.float32 else [3, 5, 5, 7, 9])
        H, W = rnd.randint(ks, 70), rnd.randint(ks, 70)
        if rnd.random() < 0.4:
            H, W = max(ks, (H + 7) // 8 * 8), max(ks, (W + 7) // 8 * 8)
        bn = max(1, int(rnd.choice([3e4, 1.5e5, 4e5]) / (H * W)))
        B = rnd.choice([1, 2, 4])
        N = max(1, bn // B)
        out.append(((B, N, H, W, D), ks, dt, rnd.choice([0, 0, 3, 4]), rnd.choice([1.0, 1.0, 0.5, D ** -0.5]), it))
    return out


@pytest.mark.parametrize("shape,ks,dtype,path,scale,seed", _cases_2d(28, 2024))
def test_random_shapes_2d(shape, ks, dtype, path, scale, seed, lib):
    prev = lib.enatten_set_path(path)
    try:
        print("case random", shape, "k=%d" % ks, dtype, "path", path, "scale", scale, flush=True)
        q, k, v, g = make_inputs(shape, dtype, seed=100 + seed)
        o, lse, dq, dk, dv = run_capi(q, k, v, g, ks, scale)
        ref = oracle_all(q, k, v, g, ks, scale)
        for name, x, r in zip(("O", "dQ", "dK", "dV"), (o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4])):
            assert torch.isfinite(x.float()).all(), name
            if dtype == torch.float32:
                assert O.max_abs_err(x, r) <= FP32_MAX_ABS, (name, O.max_abs_err(x, r))
            else:
                assert O.rel_err(x, r) <= BF16_REL, (name, O.rel_err(x, r))
        assert (lse - ref[1]).abs().max().item() <= (1e-4 if dtype == torch.float32 else 2e-2)
    finally:
        lib.enatten_set_path(prev)


def _cases_2d_narrow(n, seed):
    """Head dims that are multiples of 8 between the built ones (matrix-core kernels of the next
    of 32, 64, 128; head dims below 64 with kernel_size 11 and 13 take the general kernels)."""
    rnd = random.Random(seed)
    out = []
    for it in range(n):
        dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16])
        D = rnd.choice([8, 16, 24, 40, 48, 56, 72, 80, 88, 96, 104, 112, 120])
        ks = rnd.choice([3, 5, 5, 7, 7, 9, 11, 13])
        H, W = rnd.randint(ks, 60), rnd.randint(ks, 60)
        if rnd.random() < 0.4:
            H, W = max(ks, (H + 7) // 8 * 8), max(ks, (W + 7) // 8 * 8)
        B = rnd.choice([1, 2, 3])
        N = max(1, int(rnd.choice([2e4, 8e4, 2e5]) / (H * W)) // B)
        out.append(((B, N, H, W, D), ks, dt, rnd.choice([0, 0, 3, 4]), rnd.choice([1.0, 0.5, D ** -0.5]), it))
    return out


@pytest.mark.parametrize("shape,ks,dtype,path,scale,seed", _cases_2d_narrow(20, 31))
def test_random_shapes_2d_narrow_head_dims(shape, ks, dtype, path, scale, seed, lib):
    test_random_shapes_2d(shape, ks, dtype, path, scale, 1000 + seed, lib)


def _cases_1d(n, seed):
    rnd = random.Random(seed)
    out = []
    for it in range(n):
        dt = rnd.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        D = rnd.choice([32, 64, 128, 16])
        ks = rnd.choice([3, 5, 7, 9, 13, 17, 19, 25, 33, 49, 51])
        T = rnd.randint(ks, 700)
        B, N = rnd.choice([1, 2, 3]), rnd.choice([1, 2, 5])
        out.append(((B, N, T, D), ks, dt, it, rnd.choice([0, 4])))
    return out


@pytest.mark.parametrize("shape,ks,dtype,seed,path", _cases_1d(24, 7))
def test_random_shapes_1d(shape, ks, dtype, seed, path, lib):
    from e_natten_amd import Natten1d
    print("case random 1d", shape, "k=%d" % ks, dtype, "path", path, flush=True)
    prev = lib.enatten_set_path(path)  # 0: one-pass backward where built, 4: two passes
    try:
        _random_1d(shape, ks, dtype, seed)
    finally:
        lib.enatten_set_path(prev)


def _random_1d(shape, ks, dtype, seed):
    from e_natten_amd import Natten1d
    g = torch.Generator().manual_seed(200 + seed)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype) for _ in range(4))
    ref = O1.natten1d_explicit(q, k, v, d_o, ks)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = Natten1d.apply(qg, kg, vg, ks, 1.0)
    o.backward(d_o.cuda())
    for name, x, r in zip(("O", "dQ", "dK", "dV"), (o, qg.grad, kg.grad, vg.grad),
                          (ref[0], ref[2], ref[3], ref[4])):
        x = x.detach().cpu()
        assert torch.isfinite(x.float()).all(), name
        if dtype == torch.float32:
            assert O.max_abs_err(x, r) <= FP32_MAX_ABS, (name, O.max_abs_err(x, r))
        else:
            assert O.rel_err(x, r) <= BF16_REL, (name, O.rel_err(x, r))


def _cases_window(n, seed):
    rnd = random.Random(seed)
    out = []
    for it in range(n):
        D = rnd.choice([8, 32, 64, 128, 24])
        causal = (rnd.random() < 0.4, rnd.random() < 0.4)
        kh = rnd.choice([1, 2, 3, 4, 6, 7]) if causal[0] else rnd.choice([1, 3, 5, 7, 9])
        kw = rnd.choice([1, 2, 3, 5, 8]) if causal[1] else rnd.choice([1, 3, 5, 7, 9])
        H, W = rnd.randint(kh, 26), rnd.randint(kw, 26)
        dt = rnd.choice([torch.float32, torch.bfloat16, torch.float16])
        rpb = rnd.random() < 0.4 and not any(causal)
        out.append(((rnd.choice([1, 2]), rnd.choice([1, 3]), H, W, D), (kh, kw), causal, dt, rpb,
                    rnd.choice([1.0, 0.5, D ** -0.5]), it))
    return out


@pytest.mark.parametrize("shape,kernel,causal,dtype,with_rpb,scale,seed", _cases_window(24, 77))
def test_random_windows(shape, kernel, causal, dtype, with_rpb, scale, seed, lib):
    # rectangular and causal windows and the relative position bias against the dense-mask
    # oracle (float64 autograd), forward and backward, d_rpb included
    from e_natten_amd import natten2d
    print("case window", shape, kernel, causal, dtype, "rpb" if with_rpb else "", flush=True)
    q, k, v, g = make_inputs(shape, dtype, seed=1000 + seed, q_scale=1.0 if dtype == torch.float32 else 0.5)
    rpb = None
    if with_rpb:
        gen = torch.Generator().manual_seed(seed)
        rpb = torch.randn((shape[1], 2 * kernel[0] - 1, 2 * kernel[1] - 1), generator=gen).to(dtype)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    rr = rpb.double().requires_grad_(True) if with_rpb else None
    o_ref = O.natten2d_window_dense_mask(qr, kr, vr, kernel, causal, scale, rr)
    refs = (o_ref.detach(),) + tuple(torch.autograd.grad(o_ref, (qr, kr, vr) + ((rr,) if with_rpb else ()), g.double()))
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    rg = rpb.cuda().requires_grad_(True) if with_rpb else None
    o = natten2d(qg, kg, vg, kernel, scale, 1, causal, rg)
    outs = (o,) + tuple(torch.autograd.grad(o, (qg, kg, vg) + ((rg,) if with_rpb else ()), g.cuda()))
    for name, x, r in zip(("O", "dQ", "dK", "dV", "d_rpb"), outs, refs):
        x = x.detach().cpu()
        assert torch.isfinite(x.float()).all(), name
        if dtype == torch.float32:
            assert O.max_abs_err(x, r) <= (FP32_MAX_ABS if name != "d_rpb" else 2e-3), (name, O.max_abs_err(x, r))
        else:
            assert O.rel_err(x, r) <= (BF16_REL if name != "d_rpb" else 3e-2), (name, O.rel_err(x, r))
