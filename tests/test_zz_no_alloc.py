"""The backward entry point that allocates nothing (enatten2d_bwd_static) against
enatten2d_bwd, through the C ABI: bit-identical dQ, dK, dV on two calls in a row, the
second on a smaller input, for the kernel families that use the scratch (two-pass
matrix-core backward, general kernels) and one that does not (fused backward)."""
import pytest
import torch

from _util import ensure_built, make_inputs

BF, F32 = torch.bfloat16, torch.float32


def _both(lib, shape, dtype, ks, seed, ref_path=None):
    """dQ, dK, dV of enatten2d_bwd_static against enatten2d_bwd's, bit for bit.  `ref_path`
    forces the kernel family of the reference call (for calls whose scratch is too small
    for the family that enatten2d_bwd would pick with its own workspace)."""
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
    prev = lib.enatten_set_path(ref_path) if ref_path is not None else None
    try:
        rc = lib.enatten2d_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr(),
                               lse.data_ptr(), ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(),
                               ws.data_ptr(), B, N, H, W, D, ks, code, None, None, None, None, None,
                               1.0, st)
    finally:
        if prev is not None:
            lib.enatten_set_path(prev)
    assert rc == 0, L.last_error()

    def static_call():
        rc = lib.enatten2d_bwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                      g.data_ptr(), lse.data_ptr(), got[0].data_ptr(),
                                      got[1].data_ptr(), got[2].data_ptr(), B, N, H, W, D, ks, code,
                                      None, None, None, None, None, 1.0, st)
        assert rc == 0, L.last_error()
        torch.cuda.synchronize()

    # A first call does the one-time work of the library on this device (the lookup of the
    # scratch array's address, which may load the code object that backs it, and the
    # occupancy queries of the kernels): allocations are compared around the second call.
    static_call()
    for t in got:
        t.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info()[0]   # hipMemGetInfo: sees hipMalloc / hipFree of any library
    static_call()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed"
    for name, x, r in zip(("dQ", "dK", "dV"), got, ref):
        assert torch.isfinite(x.float()).all(), name
        assert torch.equal(x, r), "%s differs from enatten2d_bwd's" % name


@pytest.mark.gpu
@pytest.mark.parametrize("big,small,dtype,ks", [
    ((2, 4, 48, 40, 64), (1, 2, 24, 16, 64), BF, 7),      # two-pass matrix-core backward
    ((2, 2, 24, 20, 48), (1, 1, 9, 11, 48), F32, 5),      # general kernels (delta and 1/Z)
    ((1, 2, 64, 64, 128), (1, 2, 32, 40, 128), BF, 5),    # matrix-core, head_dim 128
    # float32 matrix-core backward with the scratch as its P / dS buffers (2 k^2 floats per query)
    ((1, 2, 24, 20, 64), (1, 1, 16, 16, 64), F32, 5),
])
def test_static_scratch_backward_matches(big, small, dtype, ks):
    lib = ensure_built()
    assert torch.cuda.is_available()
    print("case no-alloc", big, small, dtype, ks, flush=True)
    _both(lib, big, dtype, ks, 3)
    _both(lib, small, dtype, ks, 4)


@pytest.mark.gpu
def test_static_scratch_float32_beyond_matrix_core_buffers():
    # float32, head_dim 64, kernel_size 5: the matrix-core backward needs 2 * 25 floats per
    # query, the scratch holds 2^21 floats, so from 41944 queries on the call is served by the
    # general kernels (two floats per query); enatten2d_bwd with its own workspace would take
    # the matrix-core kernels, so the reference call is forced onto the general ones.
    from e_natten_amd import _lib as L
    lib = ensure_built()
    shape = (2, 4, 80, 72, 64)
    assert 2 * 4 * 80 * 72 * 50 > 2 * L.STATIC_BWD_MAX_QUERIES >= 2 * 2 * 4 * 80 * 72
    print("case no-alloc float32 general kernels", shape, flush=True)
    _both(lib, shape, F32, 5, 7, ref_path=L.PATH_SIMT)
    _both(lib, (1, 2, 24, 20, 64), F32, 5, 8)   # and back to the matrix-core kernels


@pytest.mark.gpu
def test_static_scratch_backward_captured_in_a_graph():
    """enatten2d_bwd_static recorded into a HIP graph after one call outside capture (the
    one-time host work of the library is not meant to run under capture), replayed three times
    with eager work in between, every replay bit-identical to enatten2d_bwd."""
    from e_natten_amd import _lib as L
    lib = ensure_built()
    shape, ks = (2, 2, 32, 24, 64), 7
    B, N, H, W, D = shape
    dev = torch.device("cuda:0")
    q, k, v, g = (t.to(dev) for t in make_inputs(shape, BF, 11))
    o = torch.empty_like(q)
    lse = torch.empty((B, N, H, W), dtype=torch.float32, device=dev)
    ws = torch.empty(lib.enatten2d_bwd_workspace_bytes(B, N, H, W, D, ks, L.BF16), dtype=torch.uint8, device=dev)
    ref = [torch.empty_like(q) for _ in range(3)]
    got = [torch.empty_like(q) for _ in range(3)]

    def fwd_and_ref(stream):
        assert lib.enatten2d_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(),
                                 B, N, H, W, D, ks, L.BF16, None, None, None, None, 1.0, stream) == 0
        assert lib.enatten2d_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), g.data_ptr(),
                                 lse.data_ptr(), ref[0].data_ptr(), ref[1].data_ptr(), ref[2].data_ptr(),
                                 ws.data_ptr(), B, N, H, W, D, ks, L.BF16, None, None, None, None, None,
                                 1.0, stream) == 0

    def static_call(stream):
        rc = lib.enatten2d_bwd_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                      g.data_ptr(), lse.data_ptr(), got[0].data_ptr(), got[1].data_ptr(),
                                      got[2].data_ptr(), B, N, H, W, D, ks, L.BF16, None, None, None,
                                      None, None, 1.0, stream)
        assert rc == 0, L.last_error()

    print("case no-alloc graph capture", shape, ks, flush=True)
    fwd_and_ref(torch.cuda.current_stream().cuda_stream)
    static_call(torch.cuda.current_stream().cuda_stream)   # outside capture first
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call(torch.cuda.current_stream().cuda_stream)
    for rep in range(3):
        # new inputs each time: the graph reads the same buffers
        q.copy_(make_inputs(shape, BF, 20 + rep)[0].to(dev))
        fwd_and_ref(torch.cuda.current_stream().cuda_stream)
        for t in got:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for name, x, r in zip(("dQ", "dK", "dV"), got, ref):
            assert torch.equal(x, r), "replay %d: %s differs from enatten2d_bwd's" % (rep, name)


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
