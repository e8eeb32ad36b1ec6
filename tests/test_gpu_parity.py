"""HIP kernels against the CPU oracle, through the C ABI, on a real MI355X.

Tolerances: float32 within 1e-4 max-abs, bfloat16/float16 within 2e-2 of the
reference's largest magnitude, on O, dQ, dK and dV.
"""
import pytest
import torch

from _util import (BF16_REL, FP32_MAX_ABS, O, assert_close, ensure_built, make_inputs,
                   oracle_all, run_capi, run_gpu)

pytestmark = pytest.mark.gpu

BF = torch.bfloat16
F32 = torch.float32
F16 = torch.float16


@pytest.fixture(scope="module", autouse=True)
def _lib():
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return ensure_built()


@pytest.fixture(params=["auto", "simt", "split"])
def path(request, _lib):
    # auto: matrix-core kernels where built (fused or two-pass backward as dispatch
    # decides); split: matrix-core kernels with the two-pass backward; simt: general kernels
    prev = _lib.enatten_set_path({"auto": 0, "simt": 1, "split": 4}[request.param])
    yield request.param
    _lib.enatten_set_path(prev)


def _case(shape, dtype, ks, seed=0, scale=1.0, q_scale=1.0, k_scale=1.0, small=False, what=""):
    q, k, v, g = make_inputs(shape, dtype, seed, q_scale, k_scale)
    print("case", what, shape, dtype, "k=%d" % ks, flush=True)
    ref = oracle_all(q, k, v, g, ks, scale, small)
    got = run_gpu(q, k, v, g, ks, scale)
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), dtype, what)
    return got, ref


def test_config1_fp32_small(path):
    # B=1, heads=2, 16x16, d=32, k=3; softmax scale d^-0.5 folded into q
    _case((1, 2, 16, 16, 32), F32, 3, seed=0, q_scale=32 ** -0.5, small=True, what="C1")


@pytest.mark.parametrize("ks", [3, 5, 7, 9, 11])
def test_reference_test_procedure(ks, path):
    # test.py:47-53: fp32 (B=2, heads=6, 16x16, d=2), loss = sum(o^2), allclose(atol=1e-5)
    from e_natten_amd import natten2d
    q, k, v, _ = make_inputs((2, 6, 16, 16, 2), F32, 0)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    p = torch.softmax(O.natten2d_qk(qr, kr, ks), dim=-1)
    o_ref = O.natten2d_av(p, vr, ks)
    (o_ref ** 2).sum().backward()
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, ks)
    (o ** 2).sum().backward()
    for x, r in ((o, o_ref), (qg.grad, qr.grad), (kg.grad, kr.grad), (vg.grad, vr.grad)):
        assert torch.allclose(x.detach().cpu().double(), r.detach(), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("side", [32, 64, 128])
def test_config2_bf16_readme_shape(side, path):
    _case((4, 4, side, side, 128), BF, 5, what="C2 side %d" % side)


@pytest.mark.parametrize("shape,dtype", [((1, 1, 8, 8, 128), BF), ((1, 2, 16, 24, 128), BF),
                                         ((4, 4, 32, 32, 128), BF), ((2, 3, 64, 40, 128), BF),
                                         ((4, 4, 128, 128, 128), BF), ((1, 3, 40, 72, 128), F16),
                                         ((2, 2, 8, 48, 128), BF), ((3, 1, 56, 8, 128), F16),
                                         ((2, 1, 16, 16, 128), BF), ((1, 2, 24, 24, 128), BF),
                                         ((20, 16, 16, 16, 128), BF),  # 80 columns per XCD: dealt in two rounds and a remainder
                                         ((1, 2, 37, 50, 128), BF)])
def test_fused_backward_path(shape, dtype, _lib):
    # the fused backward (dQ, dK, dV of every tile from one staging of q, k, v, dO),
    # forced wherever it is built, against the oracle: images that are all border (one, two and three tiles a
    # side: corner and edge tiles only), mixed, fp16, columns dealt in rounds; the last shape has sides that
    # are no multiples of 8 and is served by the two-pass kernels
    from e_natten_amd._lib import PATH_MFMA_FUSED
    prev = _lib.enatten_set_path(PATH_MFMA_FUSED)
    try:
        _case(shape, dtype, 5, what="fused backward %s" % (shape,))
    finally:
        _lib.enatten_set_path(prev)


@pytest.mark.parametrize("shape,ks,dtype", [
    ((2, 3, 56, 72, 128), 7, BF),     # one workgroup per CU, inner columns walked, then frame tiles from the counter
    ((1, 2, 64, 48, 128), 9, F16),    # frame two tiles wide
    ((1, 1, 40, 56, 128), 13, BF),    # no inner body: every tile from the counter, 12x12 blocks
    ((2, 4, 64, 72, 64), 13, BF),     # two waves per block of keys, 22x22 frame blocks, sums through LDS
    ((4, 4, 56, 56, 32), 7, BF),      # three workgroups per CU
    ((1, 2, 37, 50, 64), 5, F16),     # ragged sides
    ((1, 1, 16, 16, 128), 5, BF),     # fewer tiles than workgroups ask for
])
def test_dkdv_frame_tiles_from_the_counter(shape, ks, dtype, _lib):
    # the two-pass backward with the dK/dV pass dealing its frame tiles from the counter in
    # the workspace (automatic dispatch does so only at sizes the oracle does not reach),
    # twice in a row: the second call finds the first call's count in whatever memory it
    # gets and relies on its own dQ pass to clear it
    from e_natten_amd._lib import PATH_MFMA_SPLIT_QUEUE
    prev = _lib.enatten_set_path(PATH_MFMA_SPLIT_QUEUE)
    try:
        _case(shape, dtype, ks, what="frame tiles from the counter %s" % (shape,))
        _case(shape, dtype, ks, seed=1, what="frame tiles from the counter, second call %s" % (shape,))
    finally:
        _lib.enatten_set_path(prev)


@pytest.mark.parametrize("shape,ks,dtype", [
    ((8, 16, 16, 64, 128), 5, BF),    # several short columns per workgroup: whole columns in turn
    ((32, 8, 32, 32, 128), 5, BF),    # the same with taller columns
    ((4, 10, 128, 128, 128), 5, F16), # quarter columns in turn
    ((16, 4, 64, 64, 128), 5, BF),    # one column per workgroup
    ((8, 8, 128, 128, 128), 5, BF),   # two columns per workgroup; fused backward by default
    ((6, 7, 56, 56, 64), 7, BF),      # row-major walk (head_dim below 128), 16x8 tiles
    ((4, 8, 40, 72, 64), 9, BF),      # 16x8 tiles, last tile row half outside the image
    ((8, 8, 72, 40, 64), 13, BF),     # 16x8 tiles of eight waves (forward), ragged last tile row
    ((4, 8, 56, 88, 64), 11, F16),    # 16x8 tiles in the forward, one-halo dQ pass
    ((2, 3, 33, 47, 128), 5, BF),     # ragged sides
    ((2, 2, 24, 40, 48), 5, F32),     # general kernels
])
def test_every_output_element_is_written(shape, ks, dtype, path):
    # The outputs hold NaN before the calls (the kernels must overwrite all of them,
    # nothing is accumulated); shapes chosen for every way the tiles are dealt to the
    # workgroups.  Checked against the oracle as well.
    q, k, v, g = make_inputs(shape, dtype, seed=7)
    print("case written", shape, dtype, "k=%d" % ks, path, flush=True)
    o, lse, dq, dk, dv = run_capi(q, k, v, g, ks)
    assert torch.isfinite(lse).all(), "LSE has elements that were not written"
    ref = oracle_all(q, k, v, g, ks)
    assert_close((o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4]), dtype, "written %s" % (shape,))
    assert (lse - ref[1]).abs().max().item() <= (1e-4 if dtype == F32 else 2e-2)


def test_config2_bf16_side256():
    _case((4, 4, 256, 256, 128), BF, 5, what="C2 side 256")


@pytest.mark.parametrize("side", [64, 128])
def test_config3_fp32_readme_shape(side):
    _case((4, 4, side, side, 128), F32, 5, what="C3 side %d" % side)


@pytest.mark.parametrize("shape,ks,dtype", [((2, 4, 128, 128, 128), 7, BF), ((1, 8, 124, 140, 128), 9, torch.float16),
                                            ((1, 2, 128, 128, 128), 7, BF), ((8, 2, 112, 112, 32), 7, BF)])
def test_one_halo_in_lds_at_a_time(shape, ks, dtype, _lib):
    # head_dim 128 with kernel_size 7 and 9: the forward (from 512 tiles of 8x8 on; the
    # third shape has exactly 512) and the dQ pass stage K and V in turn in one buffer.
    # The last shape is the dQ pass of head_dim 32 compiled for three waves per SIMD.
    # Straight through the C ABI into NaN-filled buffers, against the C oracle.
    q, k, v, g = make_inputs(shape, dtype, 21)
    o, lse, dq, dk, dv = run_capi(q, k, v, g, ks)
    ref = oracle_all(q, k, v, g, ks)
    assert_close((o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4]), dtype, "one halo %s k%d" % (shape, ks))
    assert torch.isfinite(lse).all() and (lse - ref[1]).abs().max().item() <= 2e-2


@pytest.mark.parametrize("shape,ks,dtype", [
    ((2, 2, 64, 64, 128), 13, BF),      # square, inner and border tiles
    ((1, 2, 128, 128, 128), 11, BF),
    ((1, 3, 37, 29, 128), 13, F16),     # ragged sides
    ((2, 1, 45, 70, 128), 11, BF),
    ((1, 2, 13, 13, 128), 13, BF),      # window = image
    ((1, 1, 11, 40, 128), 11, F16),
    ((1, 2, 16, 24, 128), 13, BF),      # every key within reach of a border
    ((4, 8, 37, 45, 128), 13, BF),      # enough 16x8 tiles for the eight-wave forward and dQ pass, ragged
    ((3, 8, 50, 23, 128), 11, F16),     # (kernel_size 11: the forward only)
])
def test_largest_windows_at_head_dim_128(shape, ks, dtype, _lib):
    # head_dim 128 with kernel_size 11 and 13 (the reference's own test sweeps kernel sizes up to
    # 11, test.py:48): not even one workgroup's pair of halos fits LDS, so the forward and the
    # dQ pass stage one halo at a time with one workgroup per CU, and the dK/dV pass walks
    # every tile in 12x12 blocks of queries.  Through the C ABI into NaN-filled buffers.
    from e_natten_amd import kernel_path
    assert kernel_path(128, ks, dtype) == "mfma"
    q, k, v, g = make_inputs(shape, dtype, 31)
    print("case largest windows", shape, dtype, "k=%d" % ks, flush=True)
    o, lse, dq, dk, dv = run_capi(q, k, v, g, ks)
    ref = oracle_all(q, k, v, g, ks)
    assert_close((o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4]), dtype, "largest windows %s k%d" % (shape, ks))
    assert torch.isfinite(lse).all() and (lse - ref[1]).abs().max().item() <= 2e-2


@pytest.mark.parametrize("D,ks", [(32, 3), (32, 5), (32, 7), (64, 3)])
@pytest.mark.parametrize("hw", [(8, 8), (8, 21), (9, 9), (13, 16), (14, 14), (15, 17), (16, 16), (23, 31),
                                (28, 28), (40, 56), (64, 33)])
def test_one_pass_backward_small_head_dims(D, ks, hw, _lib):
    # The one-pass backward of head_dim 32 (kernel_size 3, 5, 7) and head_dim 64 (kernel_size 3),
    # forced wherever it is built (automatic dispatch takes it for small calls only): images of one
    # tile, of shifted last tiles (sides that are no multiples of 8), smaller than a staged block,
    # and with inner tiles; against the oracle and, bit for bit in dK and dV's inputs, finite
    # everywhere (outputs hold NaN beforehand).
    from e_natten_amd._lib import PATH_MFMA_FUSED
    if min(hw) < ks:
        pytest.skip("image smaller than the window")
    shape = (2, 3, hw[0], hw[1], D)
    prev = _lib.enatten_set_path(PATH_MFMA_FUSED)
    try:
        q, k, v, g = make_inputs(shape, BF, seed=5)
        print("case one-pass", shape, "k=%d" % ks, flush=True)
        o, lse, dq, dk, dv = run_capi(q, k, v, g, ks)
        ref = oracle_all(q, k, v, g, ks)
        assert_close((o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4]), BF, "one-pass %s k%d" % (shape, ks))
    finally:
        _lib.enatten_set_path(prev)


def test_one_pass_backward_fp16_and_strided_inputs(_lib):
    # fp16, and q / k / v / dO read through the strides of a fused projection
    from e_natten_amd import natten2d
    from e_natten_amd._lib import PATH_MFMA_FUSED
    prev = _lib.enatten_set_path(PATH_MFMA_FUSED)
    try:
        _case((1, 2, 30, 19, 32), F16, 7, seed=3, what="one-pass fp16")
        B, N, H, W, D = 2, 4, 24, 20, 32
        gen = torch.Generator().manual_seed(12)
        qkv = torch.randn((B, H, W, 3, N, D), generator=gen).to(BF)
        g = torch.randn((B, H, W, N, D), generator=gen).to(BF)
        q, k, v = (qkv[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
        ref = oracle_all(q.contiguous(), k.contiguous(), v.contiguous(), g.permute(0, 3, 1, 2, 4).contiguous(), 5)
        qkv_g = qkv.cuda().requires_grad_(True)
        qg, kg, vg = (qkv_g[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
        o = natten2d(qg, kg, vg, 5)
        (d_qkv,) = torch.autograd.grad(o, qkv_g, g.cuda().permute(0, 3, 1, 2, 4))
        got = (o.detach().cpu(),) + tuple(d_qkv[:, :, :, i].permute(0, 3, 1, 2, 4).cpu() for i in range(3))
        assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "one-pass strided")
    finally:
        _lib.enatten_set_path(prev)


def test_config4_large_window(path):
    _case((2, 8, 128, 128, 64), BF, 13, what="C4")


@pytest.mark.parametrize("shape,ks,dtype", [((4, 8, 41, 38, 64), 13, BF), ((4, 8, 35, 50, 64), 11, F16)])
def test_large_windows_at_head_dim_64_on_ragged_images(shape, ks, dtype, path):
    # the 16x8 tiles of the forward and of the one-halo dQ pass with a last tile that overhangs the image
    _case(shape, dtype, ks, seed=17, what="d64 large window, ragged")


@pytest.mark.parametrize("heads,side", [(2, 112), (4, 56), (8, 28), (16, 14)])
def test_config5_backbone_stages(heads, side, path):
    s = 32 ** -0.25
    _case((8, heads, side, side, 32), BF, 7, q_scale=s, k_scale=s, what="C5 %dx%d" % (side, side))


@pytest.mark.parametrize("shape,ks,dtype", [
    ((1, 1, 5, 5, 32), 5, BF),       # window == image: plain attention
    ((2, 3, 7, 19, 64), 7, BF),      # one axis equal to the window
    ((1, 2, 9, 23, 128), 5, BF),     # sides not multiples of any tile
    ((1, 2, 33, 17, 128), 3, BF),
    ((1, 2, 30, 31, 64), 9, BF),
    ((1, 1, 26, 27, 32), 11, BF),
    ((1, 1, 13, 13, 64), 13, BF),
    ((1, 2, 37, 29, 64), 13, BF),    # two waves per block of keys in the dK/dV pass, ragged sides
    ((2, 1, 43, 52, 64), 11, F16),
    ((1, 2, 16, 61, 64), 13, BF),    # 22-row frame blocks with a short axis; one-halo dQ pass
    ((1, 1, 56, 24, 64), 13, F16),   # inner tiles on one axis only
    ((1, 1, 64, 72, 64), 13, BF),    # inner tiles, second ring and border together
    ((1, 2, 48, 41, 64), 11, BF),
    ((2, 2, 12, 12, 32), 1, BF),     # k = 1: O == V
    ((1, 2, 20, 18, 64), 5, F16),
    ((1, 2, 20, 18, 128), 7, F16),
    ((1, 2, 21, 35, 128), 7, BF),    # one halo in LDS at a time (dQ pass), ragged sides
    ((1, 2, 27, 20, 128), 9, F16),
    ((2, 2, 19, 30, 32), 7, BF),     # halo tokens numbered in two blocks (10 and 12 wide)
    ((1, 2, 25, 33, 32), 9, F16),
    ((1, 3, 11, 12, 3), 3, F32),     # odd head dims: scalar loads
    ((1, 1, 9, 9, 5), 5, BF),
    ((1, 1, 10, 9, 48), 3, BF),
    ((1, 1, 8, 8, 96), 5, F32),
    ((1, 1, 8, 9, 200), 3, BF),
    ((1, 1, 6, 6, 640), 3, F32),
    ((1, 1, 16, 16, 256), 5, BF),
])
def test_edge_shapes(shape, ks, dtype, path):
    _case(shape, dtype, ks, seed=3, small=True, what="edge")


def test_scale_argument(path):
    _case((1, 2, 16, 20, 64), BF, 5, scale=0.125, small=True, what="scale")
    _case((1, 2, 12, 12, 16), F32, 3, scale=0.25, small=True, what="scale")
    # the one-kernel backward of head_dim 128, kernel_size 5 and the one-pass backward of
    # head_dim 32 form dS with the scale in it; a scale that is no power of two
    _case((1, 2, 24, 32, 128), BF, 5, scale=0.3, what="scale, fused backward")
    _case((2, 2, 16, 24, 32), BF, 7, scale=0.17, what="scale, one-pass backward")


def test_strided_qkv_views(path):
    # q, k, v as views of one fused projection output [B, H, W, 3, heads, d]
    from e_natten_amd import Natten2d
    B, N, H, W, D, ks = 2, 4, 20, 24, 64, 5
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, H, W, 3, N, D, generator=g).to(BF)
    d_o = torch.randn(B, N, H, W, D, generator=g).to(BF)
    q, k, v = (qkv[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    ref = oracle_all(q, k, v, d_o, ks, 1.0, small=True)
    fused = qkv.cuda().requires_grad_(True)
    qg, kg, vg = (fused[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    assert not qg.is_contiguous()
    # a non-contiguous upstream gradient as well
    o = Natten2d.apply(qg, kg, vg, ks)
    (o.transpose(2, 3) * d_o.cuda().transpose(2, 3)).sum().backward()
    grads = fused.grad.cpu()
    got = (o.detach().cpu(),) + tuple(grads[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "strided")


@pytest.mark.parametrize("D,ks,H,W", [(64, 5, 20, 24), (128, 5, 24, 32), (32, 7, 16, 20), (48, 3, 9, 10)])
def test_projection_layout_without_copies(D, ks, H, W, path):
    # A block's layouts either side of the operator: q, k, v are views of the fused
    # projection [B, H, W, 3, heads, d]; the output comes back in the memory order of
    # q, [B, H, W, heads, d], so merging the heads is a view; the upstream gradient
    # arrives in that order too.  None of the five tensors is copied on the way (the
    # allocator sees nothing but the outputs and the workspace), and the fused backward
    # (D = 128, sides multiples of 8) takes the strided rows as they are.
    from e_natten_amd import natten2d
    B, N = 2, 4
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, H, W, 3, N, D, generator=g).to(BF)
    d_y = torch.randn(B, H, W, N * D, generator=g).to(BF)
    q, k, v = (qkv[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    d_o = d_y.view(B, H, W, N, D).permute(0, 3, 1, 2, 4)
    ref = oracle_all(q.contiguous(), k.contiguous(), v.contiguous(), d_o.contiguous(), ks, 1.0, small=True)
    fused = qkv.cuda().requires_grad_(True)
    qg, kg, vg = (fused[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    d_y = d_y.cuda()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    o = natten2d(qg, kg, vg, ks)
    assert o.permute(0, 2, 3, 1, 4).is_contiguous(), "O is not in the memory order of q"
    y = o.permute(0, 2, 3, 1, 4).reshape(B, H, W, N * D)
    assert y.data_ptr() == o.data_ptr(), "merging the heads copied O"
    y.backward(d_y)
    torch.cuda.synchronize()
    # forward: o, lse; backward: dq, dk, dv, workspace, and autograd's gradient of the
    # projection with the three slices it accumulates: ten blocks at most
    assert torch.cuda.memory_stats()["allocation.all.allocated"] - before <= 10
    grads = fused.grad.cpu()
    got = (o.detach().cpu(),) + tuple(grads[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "projection layout D=%d" % D)


def test_fused_backward_takes_strided_rows(_lib):
    # the fused backward, forced, on views of a [B, H, W, 3, heads, d] projection and an
    # upstream gradient in [B, H, W, heads, d] order
    from e_natten_amd import natten2d
    from e_natten_amd._lib import PATH_MFMA_FUSED
    B, N, H, W, D, ks = 2, 3, 40, 32, 128, 5
    g = torch.Generator().manual_seed(6)
    qkv = torch.randn(B, H, W, 3, N, D, generator=g).to(BF)
    d_y = torch.randn(B, H, W, N, D, generator=g).to(BF)
    q, k, v = (qkv[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    ref = oracle_all(q.contiguous(), k.contiguous(), v.contiguous(),
                     d_y.permute(0, 3, 1, 2, 4).contiguous(), ks, 1.0, small=True)
    prev = _lib.enatten_set_path(PATH_MFMA_FUSED)
    try:
        fused = qkv.cuda().requires_grad_(True)
        qg, kg, vg = (fused[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
        o = natten2d(qg, kg, vg, ks)
        o.backward(d_y.cuda().permute(0, 3, 1, 2, 4))
        torch.cuda.synchronize()
    finally:
        _lib.enatten_set_path(prev)
    grads = fused.grad.cpu()
    got = (o.detach().cpu(),) + tuple(grads[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "fused backward, strided rows")


@pytest.mark.parametrize("shape,ks", [((2, 4, 16, 24, 128), 5), ((1, 2, 20, 20, 64), 7)])
def test_output_written_into_callers_layout(shape, ks, _lib):
    # straight through the C ABI: O is written into a [B, H, W, heads, D] buffer through
    # o_strides and read back from there by the backward, dO is read through do_strides
    from e_natten_amd import _lib as L
    import ctypes
    B, N, H, W, D = shape
    q, k, v, g = make_inputs(shape, BF, 9)
    ref = oracle_all(q, k, v, g, ks, small=True)
    dev = torch.device("cuda:0")
    qd, kd, vd = (t.to(dev) for t in (q, k, v))
    o_buf = torch.full((B, H, W, N, D), float("nan"), dtype=BF, device=dev)
    g_buf = g.permute(0, 2, 3, 1, 4).contiguous().to(dev)          # [B, H, W, heads, D]
    o_view, g_view = o_buf.permute(0, 3, 1, 2, 4), g_buf.permute(0, 3, 1, 2, 4)
    lse = torch.empty((B, N, H, W), dtype=torch.float32, device=dev)
    dq, dk, dv = (torch.full(shape, float("nan"), dtype=BF, device=dev) for _ in range(3))
    ws = torch.empty(_lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, ks, L.BF16), dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    so, sg = L.strides4(o_view), L.strides4(g_view)
    rc = _lib.enatten2d_fwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o_buf.data_ptr(),
                            lse.data_ptr(), B, N, H, W, D, ks, L.BF16, None, None, None, so, 1.0, st)
    assert rc == 0, L.last_error()
    rc = _lib.enatten2d_bwd(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o_buf.data_ptr(),
                            g_buf.data_ptr(), lse.data_ptr(), dq.data_ptr(), dk.data_ptr(),
                            dv.data_ptr(), ws.data_ptr(), B, N, H, W, D, ks, L.BF16, None, None,
                            None, so, sg, 1.0, st)
    assert rc == 0, L.last_error()
    torch.cuda.synchronize()
    got = (o_view.cpu(), dq.cpu(), dk.cpu(), dv.cpu())
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "O in the caller's layout")


@pytest.mark.parametrize("D,ks,hw,dtype", [
    (8, 3, (16, 16), BF), (16, 5, (24, 19), BF), (16, 13, (17, 32), F16), (24, 7, (16, 24), BF),
    (40, 5, (32, 32), BF), (48, 5, (40, 33), BF), (48, 9, (24, 40), F16), (56, 7, (19, 17), BF),
    (72, 3, (16, 16), BF), (80, 5, (32, 24), BF), (96, 7, (24, 24), F16), (96, 13, (32, 20), BF),
    (104, 9, (18, 23), BF), (120, 5, (48, 40), BF), (112, 11, (20, 20), BF),
])
def test_head_dims_between_the_built_ones(D, ks, hw, dtype, _lib):
    """Head dims that are multiples of 8 run on the matrix-core kernels of the next of 32, 64,
    128 (zero channels in LDS, the stores leave them out).  Through the C ABI, every tensor a
    [.., D] view of a buffer with 8 more channels per pixel that hold NaN (inputs) or a marker
    (outputs): the results match the oracle and not one guard channel is read or written."""
    from e_natten_amd import _lib as L, kernel_path
    assert kernel_path(D, ks, dtype) == "mfma"
    B, N, (H, W) = 2, 3, hw
    shape = (B, N, H, W, D)
    code = {BF: L.BF16, F16: L.F16}[dtype]
    q, k, v, g = make_inputs(shape, dtype, 40 + D)
    print("case narrow head dim", shape, dtype, "k=%d" % ks, flush=True)
    ref = oracle_all(q, k, v, g, ks, small=True)
    dev = torch.device("cuda:0")

    def guarded(t=None):
        buf = torch.full(shape[:-1] + (D + 8,), float("nan") if t is not None else 512.0, dtype=dtype, device=dev)
        if t is not None:
            buf[..., :D].copy_(t.to(dev))
        return buf, buf[..., :D]

    (_, qv), (_, kv), (_, vv), (_, gv) = (guarded(t) for t in (q, k, v, g))
    (ob, ov), (dqb, dqv), (dkb, dkv), (dvb, dvv) = (guarded() for _ in range(4))
    lse = torch.empty((B, N, H, W), dtype=torch.float32, device=dev)
    ws = torch.empty(_lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, ks, code), dtype=torch.uint8, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    sq, sk, sv, sg, so, sgr = (L.strides4(t) for t in (qv, kv, vv, gv, ov, dqv))
    rc = _lib.enatten2d_fwd(qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), ov.data_ptr(), lse.data_ptr(),
                            B, N, H, W, D, ks, code, sq, sk, sv, so, 1.0, st)
    assert rc == 0, L.last_error()
    rc = _lib.enatten2d_bwd_into(qv.data_ptr(), kv.data_ptr(), vv.data_ptr(), ov.data_ptr(), gv.data_ptr(),
                                 lse.data_ptr(), dqv.data_ptr(), dkv.data_ptr(), dvv.data_ptr(), ws.data_ptr(),
                                 B, N, H, W, D, ks, code, sq, sk, sv, so, sg, sgr, 1.0, st)
    assert rc == 0, L.last_error()
    torch.cuda.synchronize()
    for name, buf in (("O", ob), ("dQ", dqb), ("dK", dkb), ("dV", dvb)):
        assert (buf[..., D:].float() == 512.0).all(), "%s: a guard channel was written" % name
    got = tuple(t.float().cpu() for t in (ov, dqv, dkv, dvv))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), dtype, "head_dim %d k%d" % (D, ks))


@pytest.mark.parametrize("D,ks", [(128, 5), (64, 7), (32, 3)])
def test_misaligned_views_take_the_general_kernels(D, ks, _lib):
    # head dims the matrix-core kernels serve, but as views whose rows are not 16-byte
    # aligned (channels 4..D+4 of a wider tensor, strides that are no multiples of 8):
    # the launchers route them to the general kernels with scalar loads
    from e_natten_amd import natten2d
    shape = (1, 2, 12, 14, D)
    q, k, v, g = make_inputs(shape, BF, 13)
    ref = oracle_all(q, k, v, g, ks, small=True)
    dev = torch.device("cuda:0")
    wide = [torch.zeros(shape[:-1] + (D + 12,), dtype=BF, device=dev) for _ in range(4)]
    views = []
    for buf, t in zip(wide, (q, k, v, g)):
        view = buf[..., 4:D + 4]
        view.copy_(t.to(dev))
        views.append(view)
    assert all(t.data_ptr() % 16 != 0 and t.stride(3) % 8 != 0 for t in views)
    qg, kg, vg = (t.requires_grad_(True) for t in views[:3])
    o = natten2d(qg, kg, vg, ks)
    o.backward(views[3])
    torch.cuda.synchronize()
    got = tuple(t.detach().cpu() for t in (o, qg.grad, kg.grad, vg.grad))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "misaligned D=%d" % D)


def test_timing_aid_over_several_configurations(_lib):
    # the per-kernel event timing, switched on and off around several configurations in
    # one process, with the forward on this thread and the backward on the autograd
    # engine's thread: every timed launch is read back, and nothing is left recording
    import ctypes
    from e_natten_amd import natten2d
    cases = [((2, 2, 32, 32, 128), BF, 5), ((1, 2, 16, 16, 32), F32, 3), ((2, 4, 28, 28, 32), BF, 7),
             ((1, 2, 40, 40, 64), BF, 13)]
    for shape, dtype, ks in cases:
        q, k, v, g = (t.cuda() for t in make_inputs(shape, dtype, 1))
        q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)
        assert _lib.enatten_profile_enable(2) == 0
        for _ in range(6):
            natten2d(q, k, v, ks).backward(g)
        assert _lib.enatten_profile_enable(0) == 2
        n, ms = ctypes.c_int(), ctypes.c_double()
        seen = {}
        for slot in range(4):
            assert _lib.enatten_profile_read(slot, ctypes.byref(n), ctypes.byref(ms)) == 0
            if n.value:
                seen[_lib.enatten_profile_kernel_name(slot).decode()] = (n.value, ms.value)
        assert any(name.startswith("fwd") for name in seen), seen
        assert all(cnt == 3 and 0.0 < t < 1e3 for cnt, t in seen.values()), seen
    # off again: launches are not recorded
    natten2d(q, k, v, ks).backward(g)
    torch.cuda.synchronize()
    n, ms = ctypes.c_int(), ctypes.c_double()
    _lib.enatten_profile_read(0, ctypes.byref(n), ctypes.byref(ms))
    assert n.value == 3


def test_native_binding_is_what_runs(_lib):
    # natten2d goes through the C++ torch binding (no Python in forward or backward);
    # both bindings give bit-identical results; views, no-grad calls and inputs that
    # need no gradient behave like any torch operator
    from e_natten_amd import natten2d, ops
    assert ops.NATIVE_BINDING, "libenatten_torch.so is not built or failed to load"
    q, k, v, g = make_inputs((2, 3, 24, 40, 128), BF, 3)
    a = run_gpu(q, k, v, g, 5, binding="native")
    b = run_gpu(q, k, v, g, 5, binding="python")
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    qc, kc, vc = (t.cuda() for t in (q, k, v))
    with torch.no_grad():
        o = natten2d(qc, kc, vc, 5)
    assert not o.requires_grad and torch.equal(o.cpu(), a[0])
    with torch.inference_mode():
        assert torch.equal(natten2d(qc, kc, vc, 5).cpu(), a[0])
    kg = kc.clone().requires_grad_(True)
    o = natten2d(qc, kg, vc, 5)
    o.backward(g.cuda())
    assert torch.equal(kg.grad.cpu(), a[2]) and qc.grad is None
    # strided q, k, v and a non-contiguous upstream gradient
    B, N, H, W, D, ks = 2, 4, 20, 24, 64, 5
    gen = torch.Generator().manual_seed(5)
    qkv = torch.randn(B, H, W, 3, N, D, generator=gen).to(BF)
    d_o = torch.randn(B, N, H, W, D, generator=gen).to(BF)
    ref = oracle_all(*(qkv[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3)), d_o, ks, 1.0, small=True)
    fused = qkv.cuda().requires_grad_(True)
    qg, kg, vg = (fused[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    o = natten2d(qg, kg, vg, ks)
    (o.transpose(2, 3) * d_o.cuda().transpose(2, 3)).sum().backward()
    grads = fused.grad.cpu()
    got = (o.detach().cpu(),) + tuple(grads[:, :, :, i].permute(0, 3, 1, 2, 4) for i in range(3))
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), BF, "strided, native binding")
    # errors keep their classes
    with pytest.raises(ValueError):
        torch.ops.enatten.natten2d(qc, kc, vc, 4, 1.0)
    with pytest.raises(ValueError):
        torch.ops.enatten.na2d_bwd(qc, kc, vc, qc, torch.empty(1, device="cuda"), qc[:, :1], 5, 1.0)


def test_lse_matches_oracle(_lib):
    q, k, v, g = make_inputs((1, 2, 18, 18, 64), BF, 7)
    ref = oracle_all(q, k, v, g, 7, small=True)
    o, lse = torch.ops.enatten.na2d_fwd(q.cuda(), k.cuda(), v.cuda(), 7, 1.0)
    assert O.max_abs_err(lse.cpu(), ref[1]) < 1e-3
    q, k, v, g = make_inputs((1, 2, 10, 10, 24), F32, 7)
    ref = oracle_all(q, k, v, g, 3, small=True)
    o, lse = torch.ops.enatten.na2d_fwd(q.cuda(), k.cuda(), v.cuda(), 3, 1.0)
    assert O.max_abs_err(lse.cpu(), ref[1]) < 1e-5


def test_deterministic_bitwise(path):
    q, k, v, g = make_inputs((2, 2, 40, 40, 128), BF, 11)
    a = run_gpu(q, k, v, g, 5)
    b = run_gpu(q, k, v, g, 5)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


@pytest.mark.parametrize("dtype", [BF, F32])
def test_tensors_beyond_2_31_elements(dtype, _lib):
    # 66 x 16 images of 128 x 128 x 128: 2.2e9 elements per tensor, so the element offset of
    # the last images does not fit 31 bits and their byte offset not 32.  Inputs are drawn
    # on the GPU; images at both ends and in the middle are compared with a call on a copy
    # of that image alone, and the last image with the CPU oracle.
    from e_natten_amd import natten2d
    dev = torch.device("cuda:0")
    B, N, H, W, D = 66, 16, 128, 128, 128
    assert B * N * H * W * D > 2 ** 31
    gen = torch.Generator(device=dev).manual_seed(5)
    q, k, v, g = (torch.randn((B, N, H, W, D), device=dev, dtype=dtype, generator=gen) for _ in range(4))
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    o = natten2d(q, k, v, 5)
    grads = torch.autograd.grad(o, (q, k, v), g)
    torch.cuda.synchronize()
    for b, n in ((0, 0), (33, 7), (B - 1, N - 1)):
        qs, ks, vs = (t[b:b + 1, n:n + 1].detach().clone().requires_grad_(True) for t in (q, k, v))
        os_ = natten2d(qs, ks, vs, 5)
        gs = torch.autograd.grad(os_, (qs, ks, vs), g[b:b + 1, n:n + 1].clone())
        for name, big, small in zip(("O", "dQ", "dK", "dV"), (o,) + grads, (os_,) + gs):
            x, r = big[b:b + 1, n:n + 1].float(), small.float()
            assert torch.isfinite(x).all(), "%s of image (%d, %d) has non-finite values" % (name, b, n)
            err = (x - r).abs().max().item()
            bound = 1e-5 if dtype == F32 else 2 ** -7 * r.abs().max().item()
            assert err <= bound, "%s of image (%d, %d): %.3e > %.3e" % (name, b, n, err, bound)
    # and the last image, the one farthest beyond 2^31 elements, against the CPU oracle itself
    qc, kc, vc, gc = (t[B - 1:, N - 1:].detach().cpu() for t in (q, k, v, g))
    ref = oracle_all(qc, kc, vc, gc, 5)
    got = tuple(t[B - 1:, N - 1:].detach().cpu() for t in (o,) + grads)
    assert_close(got, (ref[0], ref[2], ref[3], ref[4]), dtype, "last image of a tensor beyond 2^31 elements")
    del q, k, v, g, o, grads
    torch.cuda.empty_cache()


@pytest.mark.parametrize("ks", [5, 7])
def test_full_size_invariants(ks):
    # properties that need no oracle, at the benchmark's full size (kernel_size 7: the size at
    # which automatic dispatch has the dK/dV pass deal its frame tiles from the counter):
    # rows of P sum to 1  => sum_keys dV == sum_queries dO
    # sum_j dS_j = 0      => dK summed over keys is zero up to rounding
    # constant V          => O equals that constant
    q, k, v, g = make_inputs((4, 4, 128, 128, 128), BF, 1)
    o, dq, dk, dv = run_gpu(q, k, v, g, ks)
    tot = g.float().sum((2, 3))
    assert ((dv.float().sum((2, 3)) - tot).abs().max() / tot.abs().max()) < 2e-2
    assert dk.float().sum((2, 3)).abs().max() / dk.float().abs().sum((2, 3)).max() < 2e-2
    vc = torch.full_like(v, 1.5)
    oc = run_gpu(q, k, vc, g, ks)[0]
    assert (oc.float() - 1.5).abs().max() < 2e-2


def test_autograd_contract(_lib):
    from e_natten_amd import Natten2d, natten2d
    q, k, v, g = make_inputs((1, 2, 12, 12, 32), F32, 2)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, 5)
    assert o.shape == q.shape and o.dtype == q.dtype and o.device == qg.device
    o.backward(g.cuda())
    assert all(t.grad is not None and t.grad.shape == q.shape for t in (qg, kg, vg))
    # default kernel size is 7, as in the reference
    o7 = natten2d(qg, kg, vg)
    ref7 = O.natten2d_gather(q.double(), k.double(), v.double(), 7)
    assert O.max_abs_err(o7.detach().cpu(), ref7) < FP32_MAX_ABS
    # no-grad call works and keeps nothing
    with torch.no_grad():
        o2 = natten2d(qg, kg, vg, 5)
    assert torch.equal(o2, o.detach())


def test_errors_on_gpu(_lib):
    from e_natten_amd import natten2d
    q = torch.randn(1, 1, 8, 8, 16, device="cuda")
    with pytest.raises(ValueError):
        natten2d(q, q, q, 4)
    with pytest.raises(ValueError):
        natten2d(q, q, q, 9)
    with pytest.raises(ValueError):
        natten2d(q, q[:, :, :4], q, 3)
    with pytest.raises(ValueError):
        natten2d(q.int(), q.int(), q.int(), 3)
    with pytest.raises(ValueError):
        natten2d(q, q.half(), q, 3)


def test_side_stream_and_graph_replay(_lib):
    # the launchers use the caller's stream and record nothing that a HIP graph
    # cannot replay: capture forward+backward once, replay it with eager work and
    # synchronisations in between, and compare every replay with the eager result
    from e_natten_amd import Natten2d
    q, k, v, g = make_inputs((2, 2, 40, 48, 64), BF, 21)
    dev = torch.device("cuda:0")
    qs, ks_, vs, gs = (t.to(dev) for t in (q, k, v, g))
    eager = run_gpu(q, k, v, g, 7)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        o, lse = torch.ops.enatten.na2d_fwd(qs, ks_, vs, 7, 1.0)
        dq, dk, dv = torch.ops.enatten.na2d_bwd(qs, ks_, vs, o, lse, gs, 7, 1.0)
    side.synchronize()
    for x, y in zip((o, dq, dk, dv), eager):
        assert torch.equal(x.cpu(), y)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o2, lse2 = torch.ops.enatten.na2d_fwd(qs, ks_, vs, 7, 1.0)
        dq2, dk2, dv2 = torch.ops.enatten.na2d_bwd(qs, ks_, vs, o2, lse2, gs, 7, 1.0)
    for _ in range(3):
        for t in (o2, dq2, dk2, dv2):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for x, y in zip((o2, dq2, dk2, dv2), eager):
            assert torch.equal(x.cpu(), y)
        _ = (qs.float() @ qs.float().transpose(-1, -2)).sum().item()  # unrelated eager work


@pytest.mark.parametrize("shape,ks,dil,dtype", [
    ((1, 2, 20, 22, 32), 3, 2, BF),      # every sub-grid on the matrix-core kernels
    ((2, 1, 31, 29, 64), 5, 3, BF),      # sub-grids of unequal sizes
    ((1, 2, 24, 24, 128), 5, 4, F16),
    ((1, 1, 14, 15, 8), 7, 2, F32),      # general kernels
])
def test_dilated_neighborhoods(shape, ks, dil, dtype, _lib):
    # natten2d(..., dilation=d) against the dense-mask oracle built from NATTEN's dilated
    # window rule (oracle/na2d_oracle.py: dilated_win_start), forward and backward
    from e_natten_amd import natten2d
    q, k, v, g = make_inputs(shape, dtype, seed=11)
    print("case dilated", shape, dtype, "k=%d dilation=%d" % (ks, dil), flush=True)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    o_ref = O.natten2d_dilated_dense_mask(qr, kr, vr, ks, dil)
    dq_ref, dk_ref, dv_ref = torch.autograd.grad(o_ref, (qr, kr, vr), g.double())
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, ks, 1.0, dil)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), g.cuda())
    assert_close(tuple(t.detach().cpu() for t in (o, dq, dk, dv)),
                 (o_ref.detach(), dq_ref, dk_ref, dv_ref), dtype, "dilated %s" % (shape,))
    with pytest.raises(ValueError):
        natten2d(qg, kg, vg, ks, 1.0, max(shape[2], shape[3]))
    # Every sub-grid is written in place, O through its strides in the forward, dQ, dK and dV
    # through enatten2d_bwd_into in the backward: the allocator sees one block per output
    # tensor, and per sub-grid only its log-sum-exp and the backward's workspace.
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    o2 = natten2d(qg, kg, vg, ks, 1.0, dil)
    grads2 = torch.autograd.grad(o2, (qg, kg, vg), g.cuda())
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] - before <= 4 + 2 * dil * dil + 1
    assert torch.equal(o2, o) and all(torch.equal(a, b) for a, b in zip(grads2, (dq, dk, dv)))


def test_traced_by_torch_compile(_lib):
    # The operators are opaque to the tracer and carry meta kernels, so a function that
    # calls them compiles as one graph (no graph break); the compiled function runs the same
    # kernels, so forward and gradients equal the eager ones bit for bit.
    from e_natten_amd import natten1d, natten2d, ops
    if not ops.NATIVE_BINDING:
        pytest.skip("native torch binding not built")

    def f(q, k, v, s):
        a = natten2d(q * 1.0, k, v, 5)
        b = natten1d(s, s, s, 7)
        return (a.float() ** 2).sum() + b.float().sum()

    q, k, v, _ = make_inputs((2, 2, 24, 24, 64), BF, seed=5)
    q, k, v = (t.cuda().requires_grad_(True) for t in (q, k, v))
    s = torch.randn(2, 2, 200, 32, device="cuda", dtype=F16, requires_grad=True)
    ref = f(q, k, v, s)
    gref = torch.autograd.grad(ref, (q, k, v, s))
    fc = torch.compile(f, backend="aot_eager", fullgraph=True)
    out = fc(q, k, v, s)
    got = torch.autograd.grad(out, (q, k, v, s))
    assert torch.equal(out.detach(), ref.detach())
    for a, b in zip(got, gref):
        assert torch.equal(a, b)


@pytest.mark.parametrize("shape,kernel,causal,dtype", [
    ((1, 2, 12, 14, 16), (3, 7), (False, False), F32),     # rectangular
    ((2, 1, 9, 20, 32), (9, 5), (False, False), BF),       # one axis fully covered
    ((1, 2, 10, 11, 8), (3, 3), (True, False), F32),       # causal rows, centred columns
    ((1, 1, 13, 9, 64), (4, 5), (True, False), F16),       # an even causal extent
    ((1, 2, 8, 12, 24), (5, 6), (True, True), F32),        # causal on both axes
    ((2, 2, 16, 16, 128), (1, 7), (False, False), BF),     # a single row per query
])
def test_rectangular_and_causal_windows(shape, kernel, causal, dtype, _lib):
    # natten2d with kernel_size = (rows, columns) and per-axis is_causal against the dense-mask
    # oracle (oracle/na2d_oracle.py: axis_window_mask), forward and backward
    from e_natten_amd import natten2d
    q, k, v, g = make_inputs(shape, dtype, seed=13)
    print("case window", shape, dtype, kernel, causal, flush=True)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    o_ref = O.natten2d_window_dense_mask(qr, kr, vr, kernel, causal, 0.5)
    dq_ref, dk_ref, dv_ref = torch.autograd.grad(o_ref, (qr, kr, vr), g.double())
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, kernel, 0.5, 1, causal)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), g.cuda())
    assert_close(tuple(t.detach().cpu() for t in (o, dq, dk, dv)),
                 (o_ref.detach(), dq_ref, dk_ref, dv_ref), dtype, "window %s %s" % (kernel, causal))


def test_square_pair_takes_the_fast_kernels(_lib):
    # kernel_size = (k, k) without causal axes is the reference's operator: same kernels, same bits
    from e_natten_amd import natten2d
    q, k, v, _ = make_inputs((1, 2, 16, 16, 128), BF, seed=3)
    q, k, v = (t.cuda() for t in (q, k, v))
    assert torch.equal(natten2d(q, k, v, (5, 5)), natten2d(q, k, v, 5))
    assert torch.equal(natten2d(q, k, v, 5, is_causal=(False, False)), natten2d(q, k, v, 5))


def test_causal_window_with_dilation(_lib):
    from e_natten_amd import natten2d
    shape, kernel, causal, dil = (1, 2, 12, 13, 16), (3, 3), (False, True), 2
    q, k, v, g = make_inputs(shape, F32, seed=17)
    qr, kr, vr = (t.double().requires_grad_(True) for t in (q, k, v))
    # oracle: the undilated rule on each of the dilation^2 sub-grids
    o_ref = torch.empty(shape, dtype=torch.float64)
    for i in range(dil):
        for j in range(dil):
            sub = (slice(None), slice(None), slice(i, None, dil), slice(j, None, dil))
            o_ref[sub] = O.natten2d_window_dense_mask(qr[sub], kr[sub], vr[sub], kernel, causal)
    ref = torch.autograd.grad(o_ref, (qr, kr, vr), g.double())
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, kernel, 1.0, dil, causal)
    got = torch.autograd.grad(o, (qg, kg, vg), g.cuda())
    assert_close(tuple(t.detach().cpu() for t in (o, *got)), (o_ref.detach(), *ref), F32, "dilated causal")


@pytest.mark.parametrize("shape,kernel,dtype,dil", [
    ((2, 3, 10, 12, 16), (3, 3), F32, 1),
    ((1, 2, 9, 14, 32), (5, 3), BF, 1),
    ((1, 2, 16, 16, 128), (5, 5), F16, 1),     # a square window with a bias: general kernels
    ((1, 2, 13, 12, 8), (3, 3), F32, 2),       # with dilation: the bias gradient sums over sub-grids
])
def test_relative_position_bias(shape, kernel, dtype, dil, _lib):
    # natten2d(..., rpb=...) against the dense-mask oracle with the bias in the mask; O, dQ,
    # dK, dV and the bias gradient, which is summed in a fixed order: a second backward gives
    # the same bits
    from e_natten_amd import natten2d
    q, k, v, g = make_inputs(shape, dtype, seed=19)
    gen = torch.Generator().manual_seed(3)
    rpb = torch.randn(shape[1], 2 * kernel[0] - 1, 2 * kernel[1] - 1, generator=gen).to(dtype)
    print("case rpb", shape, dtype, kernel, "dilation", dil, flush=True)
    qr, kr, vr, br = (t.double().requires_grad_(True) for t in (q, k, v, rpb))
    o_ref = torch.empty(shape, dtype=torch.float64)
    for i in range(dil):
        for j in range(dil):
            sub = (slice(None), slice(None), slice(i, None, dil), slice(j, None, dil))
            o_ref[sub] = O.natten2d_window_dense_mask(qr[sub], kr[sub], vr[sub], kernel, scale=0.4, rpb=br)
    ref = torch.autograd.grad(o_ref, (qr, kr, vr, br), g.double())
    qg, kg, vg, bg = (t.cuda().requires_grad_(True) for t in (q, k, v, rpb))
    o = natten2d(qg, kg, vg, kernel, 0.4, dil, False, bg)
    got = torch.autograd.grad(o, (qg, kg, vg, bg), g.cuda())
    assert_close(tuple(t.detach().cpu() for t in (o, *got[:3])), (o_ref.detach(), *ref[:3]), dtype, "rpb")
    d_rpb, d_ref = got[3].detach().cpu(), ref[3]
    assert d_rpb.shape == rpb.shape and d_rpb.dtype == dtype
    err = (O.max_abs_err(d_rpb, d_ref) / max(1.0, d_ref.abs().max().item()) if dtype == F32
           else O.rel_err(d_rpb, d_ref))
    print("   d_rpb err %.3e" % err, flush=True)
    assert err <= (1e-4 if dtype == F32 else BF16_REL)
    again = torch.autograd.grad(natten2d(qg, kg, vg, kernel, 0.4, dil, False, bg), (qg, kg, vg, bg), g.cuda())
    assert all(torch.equal(a, b) for a, b in zip(again, got)), "the bias gradient is not bit-reproducible"


@pytest.mark.parametrize("shape,ks", [((2, 3, 8, 2), 7), ((1, 2, 11, 5), 3)])
def test_float64_gradcheck_1d(shape, ks, _lib):
    # the reference's own gradient check (gradcheck.py:6-15: float64 (2, 3, 8, 2), kernel_size 7,
    # eps 1e-6, atol 1e-4), run on this operator itself
    from e_natten_amd import natten1d
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(shape, generator=g, dtype=torch.float64).cuda().requires_grad_(True) for _ in range(3))
    print("case float64 gradcheck 1d", shape, ks, flush=True)
    assert torch.autograd.gradcheck(lambda a, b, c: natten1d(a, b, c, ks), (q, k, v), eps=1e-6, atol=1e-4)


@pytest.mark.parametrize("shape,ks", [((1, 2, 6, 7, 3), 3), ((2, 1, 5, 5, 2), 5), ((1, 1, 9, 8, 4), 7)])
def test_float64_gradcheck_2d(shape, ks, _lib):
    from e_natten_amd import natten2d
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(shape, generator=g, dtype=torch.float64).cuda().requires_grad_(True) for _ in range(3))
    print("case float64 gradcheck 2d", shape, ks, flush=True)
    assert torch.autograd.gradcheck(lambda a, b, c: natten2d(a, b, c, ks, 0.7), (q, k, v), eps=1e-6, atol=1e-4)


@pytest.mark.parametrize("shape,ks", [((2, 2, 16, 13, 24), 5), ((1, 2, 20, 20, 130), 3), ((1, 1, 9, 9, 8), 9)])
def test_float64_against_the_oracle(shape, ks, _lib):
    # float64 tensors in plain double arithmetic: agreement with the float64 oracle to 1e-10
    from e_natten_amd import natten2d
    g = torch.Generator().manual_seed(2)
    q, k, v, d_o = (torch.randn(shape, generator=g, dtype=torch.float64) for _ in range(4))
    ref = O.natten2d_explicit(q, k, v, d_o, ks, 1.0, compute_dtype=torch.float64)
    qg, kg, vg = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = natten2d(qg, kg, vg, ks)
    dq, dk, dv = torch.autograd.grad(o, (qg, kg, vg), d_o.cuda())
    for name, x, r in zip(("O", "dQ", "dK", "dV"), (o, dq, dk, dv), (ref[0], ref[2], ref[3], ref[4])):
        err = (x.detach().cpu() - r.double()).abs().max().item()
        print("   float64", name, "max-abs err %.2e" % err, flush=True)
        assert err <= 1e-10 * max(1.0, r.abs().max().item()), (name, err)
