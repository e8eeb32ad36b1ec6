"""1D operator (natten1d) on the GPU against the CPU oracle, through the C ABI."""
import pytest
import torch

from _util import BF16_REL, FP32_MAX_ABS, O, ensure_built
from oracle import na1d_oracle as O1
from oracle import na2d_c

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _lib():
    assert torch.cuda.is_available()
    return ensure_built()


@pytest.fixture(params=["auto", "split"])
def path(request, _lib):
    # auto: the one-pass backward where it is built; split: always the dQ and dK/dV passes
    prev = _lib.enatten_set_path({"auto": 0, "split": 4}[request.param])
    yield request.param
    _lib.enatten_set_path(prev)


def _run(shape, dtype, ks, seed=0, scale=1.0):
    from e_natten_amd import Natten1d
    g = torch.Generator().manual_seed(seed)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype) for _ in range(4))
    ref = O1.natten1d_explicit(q, k, v, d_o, ks, scale)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = Natten1d.apply(qg, kg, vg, ks, scale)
    o.backward(d_o.cuda())
    got = tuple(t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad))
    for name, x, r in zip(("O", "dQ", "dK", "dV"), got, (ref[0], ref[2], ref[3], ref[4])):
        err = O.max_abs_err(x, r) if dtype == torch.float32 else O.rel_err(x, r)
        tol = FP32_MAX_ABS if dtype == torch.float32 else BF16_REL
        print("   1d", shape, dtype, "k=%d" % ks, name, "err %.3e" % err, flush=True)
        assert err <= tol, (name, err)
    return got, ref


@pytest.mark.parametrize("ks", [3, 5, 7, 9, 11])
def test_reference_test_procedure_1d(ks):
    # test.py:51: fp32 (B=2, heads=3, T=16, d=2), loss sum(o^2), allclose(atol=1e-5)
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn((2, 3, 16, 2), generator=g) for _ in range(3))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    o_ref = O1.natten1d_gather(qr, kr, vr, ks)
    (o_ref ** 2).sum().backward()
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten1d(qg, kg, vg, ks)
    (o ** 2).sum().backward()
    for x, r in ((o, o_ref), (qg.grad, qr.grad), (kg.grad, kr.grad), (vg.grad, vr.grad)):
        assert torch.allclose(x.detach().cpu().double(), r.detach(), atol=1e-5, rtol=1e-5)


def test_gradcheck_shape_of_reference():
    # gradcheck.py:6-15 checks (2, 3, 8, 2), k=7 in double; float32 here against the fp64 oracle
    _run((2, 3, 8, 2), torch.float32, 7, seed=1)


@pytest.mark.parametrize("shape,ks,dtype", [
    ((2, 4, 1024, 64), 7, torch.bfloat16),
    ((1, 2, 333, 128), 13, torch.bfloat16),
    ((1, 2, 50, 32), 5, torch.float16),
    ((2, 2, 257, 48), 9, torch.float32),
    ((1, 1, 7, 8), 7, torch.float32),      # window == sequence
    ((1, 3, 19, 5), 3, torch.float32),     # odd head dim
    ((1, 2, 40, 16), 1, torch.bfloat16),
    ((2, 2, 64, 128), 3, torch.bfloat16),    # exactly one tile
    ((1, 3, 65, 64), 17, torch.bfloat16),    # a second tile of one position; largest 32-token window
    ((1, 2, 200, 32), 19, torch.float16),    # 64-token windows
    ((1, 1, 130, 64), 49, torch.bfloat16),   # largest window of the matrix-core kernels
    ((1, 1, 49, 128), 49, torch.bfloat16),   # window == sequence
    ((1, 2, 300, 128), 31, torch.bfloat16),
    ((3, 2, 1000, 32), 5, torch.bfloat16),
    ((1, 1, 120, 64), 51, torch.bfloat16),   # beyond them: general kernels
    ((1, 2, 1 << 18, 32), 7, torch.bfloat16),  # a long sequence: 4096 tiles per (batch, head)
])
def test_shapes_1d(shape, ks, dtype, path):
    _run(shape, dtype, ks, seed=2)


@pytest.mark.parametrize("D,ks,T,dtype", [
    (8, 3, 70, torch.bfloat16), (16, 7, 200, torch.bfloat16), (24, 13, 129, torch.float16),
    (40, 5, 64, torch.bfloat16), (48, 33, 300, torch.bfloat16), (56, 17, 65, torch.bfloat16),
    (72, 7, 500, torch.float16), (96, 19, 150, torch.bfloat16), (96, 49, 260, torch.bfloat16),
    (120, 3, 33, torch.bfloat16), (104, 25, 400, torch.bfloat16),
])
def test_head_dims_between_the_built_ones_1d(D, ks, T, dtype, path, _lib):
    """Head dims that are multiples of 8 run on the 1D matrix-core kernels of the next of 32, 64,
    128.  Through the C ABI, every tensor a [.., D] view of a buffer with 8 more channels per
    position (NaN beside the inputs, a marker beside the outputs): results against the oracle,
    and no guard channel read or written."""
    from e_natten_amd import _lib as L
    B, N = 2, 3
    shape = (B, N, T, D)
    code = {torch.bfloat16: L.BF16, torch.float16: L.F16}[dtype]
    g = torch.Generator().manual_seed(70 + D)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype) for _ in range(4))
    print("case narrow head dim 1d", shape, dtype, "k=%d" % ks, path, flush=True)
    ref = O1.natten1d_explicit(q, k, v, d_o, ks, 1.0)
    dev = torch.device("cuda:0")

    def guarded(t=None):
        buf = torch.full(shape[:-1] + (D + 8,), float("nan") if t is not None else 512.0, dtype=dtype, device=dev)
        if t is not None:
            buf[..., :D].copy_(t.to(dev))
        return buf, buf[..., :D]

    (_, qv), (_, kv), (_, vv), (_, gv) = (guarded(t) for t in (q, k, v, d_o))
    (ob, ov), (dqb, dqv), (dkb, dkv), (dvb, dvv) = (guarded() for _ in range(4))
    lse = torch.empty((B, N, T), dtype=torch.float32, device=dev)
    ws = torch.empty(_lib.enatten1d_bwd_workspace_bytes(B, N, T), dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    sq, sk, sv, sg, so, sgr = (L.strides3(t) for t in (qv, kv, vv, gv, ov, dqv))
    rc = _lib.enatten1d_fwd(qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), ov.data_ptr(), lse.data_ptr(),
                            B, N, T, D, ks, code, sq, sk, sv, so, 1.0, st)
    assert rc == 0, L.last_error()
    rc = _lib.enatten1d_bwd_into(qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), ov.data_ptr(), gv.data_ptr(),
                                 lse.data_ptr(), dqv.data_ptr(), dkv.data_ptr(), dvv.data_ptr(), ws.data_ptr(),
                                 B, N, T, D, ks, code, sq, sk, sv, so, sg, sgr, 1.0, st)
    assert rc == 0, L.last_error()
    torch.cuda.synchronize()
    for name, buf in (("O", ob), ("dQ", dqb), ("dK", dkb), ("dV", dvb)):
        assert (buf[..., D:].float() == 512.0).all(), "%s: a guard channel was written" % name
    for name, x, r in zip(("O", "dQ", "dK", "dV"), (ov, dqv, dkv, dvv), (ref[0], ref[2], ref[3], ref[4])):
        x = x.float().cpu()
        assert torch.isfinite(x).all(), name
        assert O.rel_err(x, r) <= BF16_REL, (name, O.rel_err(x, r))


def test_scale_and_c_oracle_1d():
    got, ref = _run((2, 2, 100, 64), torch.float32, 5, seed=3, scale=0.125)
    g = torch.Generator().manual_seed(3)
    q, k, v, d_o = (torch.randn((2, 2, 100, 64), generator=g) for _ in range(4))
    oc, _ = na2d_c.forward_1d(q, k, v, 5, 0.125)
    assert O.max_abs_err(got[0], oc) < FP32_MAX_ABS


def test_strided_and_contract_1d():
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(2, 64, 3, 4, 32, generator=g).to(torch.bfloat16)  # [B, T, 3, heads, d]
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    ref = O1.natten1d_gather(q.double(), k.double(), v.double(), 7)
    dev = qkv.cuda()
    o = natten1d(*(dev[:, :, i].permute(0, 2, 1, 3) for i in range(3)), 7)
    assert o.shape == q.shape and o.dtype == torch.bfloat16
    assert O.rel_err(o.cpu(), ref) < BF16_REL
    with pytest.raises(ValueError):
        natten1d(dev[:, :, 0], dev[:, :, 1], dev[:, :, 2], 4)


@pytest.mark.parametrize("shape,ks,dil,dtype", [((2, 2, 150, 64), 7, 3, torch.bfloat16),
                                                ((1, 3, 61, 16), 5, 2, torch.float32)])
def test_dilated_1d(shape, ks, dil, dtype):
    # against a dense banded mask built from NATTEN's dilated window rule
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(6)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype) for _ in range(4))
    T = shape[2]
    m = torch.zeros(T, T, dtype=torch.bool)
    for i in range(T):
        s0 = O.dilated_win_start(i, T, ks, dil)
        m[i, s0:s0 + ks * dil:dil] = True
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    o_ref = torch.nn.functional.scaled_dot_product_attention(qr, kr, vr, attn_mask=m, scale=1.0)
    refs = (o_ref,) + torch.autograd.grad(o_ref, (qr, kr, vr), d_o.double())
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten1d(qg, kg, vg, ks, 1.0, dil)
    got = (o,) + torch.autograd.grad(o, (qg, kg, vg), d_o.cuda())
    for name, x, r in zip(("O", "dQ", "dK", "dV"), got, refs):
        x, r = x.detach().cpu(), r.detach()
        err = O.max_abs_err(x, r) if dtype == torch.float32 else O.rel_err(x, r)
        assert err <= (FP32_MAX_ABS if dtype == torch.float32 else BF16_REL), (name, err)


@pytest.mark.parametrize("shape,ks,dtype", [((2, 2, 100, 32), 7, torch.float32),
                                            ((1, 3, 257, 64), 16, torch.bfloat16),
                                            ((2, 2, 48, 16), 48, torch.float32)])
def test_causal_1d(shape, ks, dtype):
    # natten1d(..., is_causal=True): query t attends keys max(t - ks + 1, 0) .. t; against the
    # dense-mask oracle, and for ks = T against torch's own causal attention
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(23)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype) for _ in range(4))
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    o_ref = O.natten2d_window_dense_mask(qr.unsqueeze(2), kr.unsqueeze(2), vr.unsqueeze(2), (1, ks),
                                         (False, True), 0.25).squeeze(2)
    ref = (o_ref.detach(), *torch.autograd.grad(o_ref, (qr, kr, vr), d_o.double()))
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten1d(qg, kg, vg, ks, 0.25, 1, True)
    got = (o.detach().cpu(), *(t.cpu() for t in torch.autograd.grad(o, (qg, kg, vg), d_o.cuda())))
    for name, x, r in zip(("O", "dQ", "dK", "dV"), got, ref):
        err = O.max_abs_err(x, r) if dtype == torch.float32 else O.rel_err(x, r)
        print("   causal 1d", shape, dtype, "k=%d" % ks, name, "err %.3e" % err, flush=True)
        assert err <= (FP32_MAX_ABS if dtype == torch.float32 else BF16_REL), (name, err)
    if ks == shape[2]:
        sdpa = torch.nn.functional.scaled_dot_product_attention(qg, kg, vg, is_causal=True, scale=0.25)
        assert (o - sdpa).abs().max().item() < 1e-4


def test_rpb_1d():
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(29)
    shape, ks = (2, 3, 77, 16), 7
    q, k, v, d_o = (torch.randn(shape, generator=g) for _ in range(4))
    rpb = torch.randn(3, 2 * ks - 1, generator=g)
    qr, kr, vr, br = (t.double().requires_grad_(True) for t in (q, k, v, rpb))
    o_ref = O.natten2d_window_dense_mask(qr.unsqueeze(2), kr.unsqueeze(2), vr.unsqueeze(2), (1, ks),
                                         rpb=br.unsqueeze(1)).squeeze(2)
    ref = (o_ref.detach(), *torch.autograd.grad(o_ref, (qr, kr, vr, br), d_o.double()))
    qg, kg, vg, bg = (t.cuda().requires_grad_(True) for t in (q, k, v, rpb))
    o = natten1d(qg, kg, vg, ks, rpb=bg)
    got = (o.detach().cpu(), *(t.cpu() for t in torch.autograd.grad(o, (qg, kg, vg, bg), d_o.cuda())))
    for name, x, r in zip(("O", "dQ", "dK", "dV", "dRPB"), got, ref):
        err = O.max_abs_err(x, r) / max(1.0, r.abs().max().item())
        print("   rpb 1d", name, "err %.3e" % err, flush=True)
        assert err <= FP32_MAX_ABS, (name, err)


def test_sequences_beyond_2_31_elements(_lib):
    # 66 x 16 sequences of 16384 x 128: 2.2e9 elements per tensor; sequences at both ends and
    # in the middle against a call on a copy of that sequence alone
    from e_natten_amd import natten1d
    dev = torch.device("cuda:0")
    B, N, T, D = 66, 16, 16384, 128
    assert B * N * T * D > 2 ** 31
    gen = torch.Generator(device=dev).manual_seed(6)
    q, k, v, g = (torch.randn((B, N, T, D), device=dev, dtype=torch.bfloat16, generator=gen) for _ in range(4))
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    o = natten1d(q, k, v, 13)
    grads = torch.autograd.grad(o, (q, k, v), g)
    torch.cuda.synchronize()
    for b, n in ((0, 0), (33, 7), (B - 1, N - 1)):
        qs, ks, vs = (t[b:b + 1, n:n + 1].detach().clone().requires_grad_(True) for t in (q, k, v))
        os_ = natten1d(qs, ks, vs, 13)
        gs = torch.autograd.grad(os_, (qs, ks, vs), g[b:b + 1, n:n + 1].clone())
        for name, big, small in zip(("O", "dQ", "dK", "dV"), (o,) + grads, (os_,) + gs):
            x, r = big[b:b + 1, n:n + 1].float(), small.float()
            assert torch.isfinite(x).all()
            err = (x - r).abs().max().item()
            assert err <= 2 ** -7 * r.abs().max().item(), "%s of sequence (%d, %d): %.3e" % (name, b, n, err)
    del q, k, v, g, o, grads
    torch.cuda.empty_cache()

