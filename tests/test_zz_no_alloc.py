"""The backward entry point that allocates nothing (enatten2d_bwd_static) against
enatten2d_bwd, through the C ABI: bit-identical dQ, dK, dV on two calls in a row, the
second on a smaller input, for the kernel families that use the scratch (two-pass
matrix-core backward, general kernels) and one that does not (fused backward)."""
import pytest
import torch

from _util import ensure_built, make_inputs

BF, F32 = torch.bfloat16, torch.float32


def _both(lib, shape, dtype, ks, seed):
    from e_natten_amd import _lib as L
    code = {F32: L.F32, BF: L.BF16}[dtype]
    B, N, H, W, D = shape
    dev = torch.device("cuda:0")
    q, k, v, g = (t.to(dev) for t in make_inputs(shape, dtype, seed))
    o = torch.empty_like(q)
    lse = torch.empty((B, N, H, W), dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.enatten2d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                           B, N, H, W, D, ks, code, None, None, None, None, 1.0, st)
    assert rc == 0, L.last_error()
    ws = torch.empty(lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, ks, code), dtype=torch.uint8, device=dev)
    ref = [torch.full_like(q, float("nan")) for _ in range(3)]
    got = [torch.full_like(q, float("nan")) for _ in range(3)]
    rc = lib.enatten2d_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr(),
                           lse.data_ptr(), ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(),
                           ws.data_ptr(), B, N, H, W, D, ks, code, None, None, None, None, None,
                           1.0, st)
    assert rc == 0, L.last_error()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    rc = lib.enatten2d_bwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                  g.data_ptr(), lse.data_ptr(), got[0].data_ptr(),
                                  got[1].data_ptr(), got[2].data_ptr(), B, N, H, W, D, ks, code,
                                  None, None, None, None, None, 1.0, st)
    assert rc == 0, L.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    for name, x, r in zip(("dQ", "dK", "dV"), got, ref):
        assert torch.isfinite(x.float()).all(), name
        assert torch.equal(x, r), "%s differs from enatten2d_bwd's" % name


@pytest.mark.gpu
@pytest.mark.parametrize("big,small,dtype,ks", [
    ((2, 4, 48, 40, 64), (1, 2, 24, 16, 64), BF, 7),      # two-pass matrix-core backward
    ((2, 2, 24, 20, 48), (1, 1, 9, 11, 48), F32, 5),      # general kernels (delta and 1/Z)
    ((1, 2, 64, 64, 128), (1, 2, 32, 40, 128), BF, 5),    # matrix-core, head_dim 128
])
def test_static_scratch_backward_matches(big, small, dtype, ks):
    lib = ensure_built()
    assert torch.cuda.is_available()
    print("case no-alloc", big, small, dtype, ks, flush=True)
    _both(lib, big, dtype, ks, 3)
    _both(lib, small, dtype, ks, 4)


@pytest.mark.gpu
def test_static_scratch_backward_fused_path_and_limit():
    from e_natten_amd import _lib as L
    lib = ensure_built()
    prev = lib.enatten_set_path(L.PATH_MFMA_FUSED)
    try:
        _both(lib, (1, 2, 32, 32, 128), BF, 5, 5)
        _both(lib, (1, 1, 16, 24, 128), BF, 5, 6)
    finally:
        lib.enatten_set_path(prev)


def test_static_scratch_backward_rejects_large_calls():
    # more queries than the built-in scratch holds: refused before anything is touched
    from e_natten_amd import _lib as L
    lib = ensure_built()
    side = 1024
    assert 2 * side * side > L.STATIC_BWD_MAX_QUERIES
    rc = lib.enatten2d_bwd_static(1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 2, side, side, 64, 5, L.BF16, None,
                                  None, None, None, None, 1.0, None)
    assert rc == 2 and "scratch" in L.last_error()
    assert lib.enatten2d_bwd_static(1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 8, 8, 64, 4, L.BF16, None, None,
                                    None, None, None, 1.0, None) == 1
