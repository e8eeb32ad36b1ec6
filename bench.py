"""Benchmark of the fused 2D neighborhood attention hot path on one MI355X.

A step is one forward + backward of ``natten2d`` (through the autograd Function
and the C ABI) on the reference's benchmark shape (bench.py:14,39 of the
reference: B=4, heads=4, head_dim=128, kernel_size=5) in bf16 at image side 128.
Prints ONE JSON line.  `value` is useful TFLOP/s (14*k^2*d FLOP per query);
`roofline` is the achieved algorithmic HBM bandwidth of the slowest kernel, from
HIP events recorded around kernel launches inside the timed region;
`cpu_baseline` times the CPU restatement of the reference's algorithm on this
machine's host cores on a bounded sample of the same workload.

Cold and hot: the timed steps rotate over several sets of q, k, v, dO that together
exceed twice the 256 MB memory-side cache, so every step finds its inputs in HBM
(the reference's triton.testing.do_bench, its bench.py:28,59, flushes the cache
between iterations for the same reason); `hot_ms_per_step` repeats one set.  The
sweep rows say whether their working set fits that cache.  `unfused_gpu` times the
unfused qk -> softmax -> av formulation in plain torch on the GPU, the comparator of
the reference's benchmark (its bench.py:23,51-56 uses NATTEN's unfused ops).
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_PEAK_TF = {"bf16": 2500.0, "fp16": 2500.0}   # dense matrix-core peaks, published
MALL_BYTES = 256 << 20       # memory-side (Infinity) cache
KERNELS = ("fwd", "bwd_dq", "bwd_dkdv", "bwd_fused")


def rotating_sets(shape, dtype, dev, tensors_per_set, seed=0, max_sets=600):
    """Enough sets of `tensors_per_set` random tensors of `shape`, carved out of one
    allocation, to exceed twice the memory-side cache (at least 3 sets).  Returns the
    list of sets and whether their total really exceeds that bound."""
    import torch
    numel = 1
    for x in shape:
        numel *= x
    esize = torch.empty((), dtype=dtype).element_size()
    set_bytes = tensors_per_set * numel * esize
    n = min(max_sets, max(3, -(-2 * MALL_BYTES // set_bytes) + 1))
    g = torch.Generator(device=dev).manual_seed(seed)
    big = torch.randn((n, tensors_per_set) + tuple(shape), generator=g, device=dev,
                      dtype=torch.float32 if n * set_bytes < (8 << 30) else dtype).to(dtype)
    return [tuple(big[i, j] for j in range(tensors_per_set)) for i in range(n)], \
        n * set_bytes > 2 * MALL_BYTES


def unfused_gpu(q, k, v, d_o, ks, iters=5):
    """The unfused formulation on the GPU in plain torch, as NATTEN's qk / av ops
    compute it (the reference's comparator, its bench.py:23 and :51-56): gather every
    query's k*k keys, logits, softmax, gather the values, weighted sum; backward by
    autograd.  Wall-clock per forward and per forward+backward."""
    import torch
    B, N, H, W, D = q.shape
    dev = q.device
    ar = lambda L: (torch.arange(L, device=dev) - ks // 2).clamp(0, L - ks)
    rows = ar(H)[:, None] + torch.arange(ks, device=dev)[None, :]            # [H, k]
    cols = ar(W)[:, None] + torch.arange(ks, device=dev)[None, :]            # [W, k]
    idx = (rows[:, None, :, None] * W + cols[None, :, None, :]).reshape(H, W, ks * ks)

    def fwd(q, k, v):
        kg = k.flatten(2, 3)[:, :, idx]                                     # [B, N, H, W, k*k, D]
        p = torch.softmax(torch.einsum("bnhwd,bnhwjd->bnhwj", q, kg).float(), dim=-1).to(q.dtype)
        return torch.einsum("bnhwj,bnhwjd->bnhwd", p, v.flatten(2, 3)[:, :, idx])

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / iters

    with torch.no_grad():
        fwd_ms = timed(lambda: fwd(q, k, v))
    qq, kk, vv = (t.detach().requires_grad_(True) for t in (q, k, v))
    step_ms = timed(lambda: torch.autograd.grad(fwd(qq, kk, vv), (qq, kk, vv), d_o))
    return {"fwd_ms": fwd_ms, "ms_per_step": step_ms,
            "what": "torch gather + einsum + softmax on the GPU, %s" % str(q.dtype).replace("torch.", "")}


def algorithmic_bytes(B, N, H, W, D, esize):
    """Bytes each kernel must move at minimum, per launch.
    fwd : read q,k,v, write o (+ 4 B/query log-sum-exp)
    dq  : read q,k,v,dO (+ lse), write dq
    dkdv: read q,k,v,dO (+ lse), write dk,dv
    fused backward: read q,k,v,dO (+ lse), write dq,dk,dv
    path: 11*M*s + 8*q, the fused-backward minimum (q,k,v,dO read once in bwd)."""
    q = B * N * H * W
    M = q * D * esize
    return {"fwd": 4 * M + 4 * q, "bwd_dq": 5 * M + 4 * q, "bwd_dkdv": 6 * M + 4 * q,
            "bwd_fused": 7 * M + 4 * q, "path": 11 * M + 8 * q}


def cpu_baseline(shape, ks, dtype, useful_flop, budget_rows=8):
    """Times the CPU restatements on this host.  The headline figure is the
    loop port of the reference's algorithm (its Python loops, softmax Jacobian
    and inverse-neighbourhood gather) on a band of image rows, scaled to the
    whole image; the vectorised and C/OpenMP oracles are timed on the full
    workload beside it."""
    import torch
    from oracle import na2d_c, na2d_oracle as O
    B, N, H, W, D = shape
    g = torch.Generator().manual_seed(0)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype).float() for _ in range(4))
    cores = os.cpu_count() or 1
    torch.set_num_threads(min(cores, 16))
    threads = torch.get_num_threads()

    r0 = (H // 2) - (H // 2) % 3
    r1 = min(H, r0 + budget_rows)
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    t0 = time.perf_counter()
    o = O.natten2d_loops(qq, kk, vv, ks, (r0, r1))
    o.backward(d_o)
    loops_s = (time.perf_counter() - t0) * H / (r1 - r0)

    t0 = time.perf_counter()
    O.natten2d_gather_grads(q, k, v, d_o, ks, compute_dtype=torch.float32)
    vec_s = time.perf_counter() - t0

    na2d_c.lib()
    t0 = time.perf_counter()
    na2d_c.forward(q, k, v, ks, nthreads=threads)
    na2d_c.backward(q, k, v, d_o, ks, nthreads=threads)
    c_s = time.perf_counter() - t0

    # The loop port on a WHOLE configuration that it finishes in seconds, nothing scaled:
    # the same batch, heads, head_dim and kernel_size on 32x32 images.
    whole = None
    if H >= 32 and W >= 32:
        ws = (B, N, 32, 32, D)
        wq, wk, wv, wg = (torch.randn(ws, generator=g).to(dtype).float() for _ in range(4))
        wq, wk, wv = (t.requires_grad_(True) for t in (wq, wk, wv))
        t0 = time.perf_counter()
        O.natten2d_loops(wq, wk, wv, ks).backward(wg)
        whole = {"workload": "B=%d heads=%d H=W=32 head_dim=%d kernel_size=%d, all rows" % (B, N, D, ks),
                 "ms": (time.perf_counter() - t0) * 1e3}
    return {
        "loop_port_whole_config": whole,
        "value": useful_flop / loops_s / 1e12, "unit": "TFLOP/s", "cores": threads,
        "kind": "port", "ms": loops_s * 1e3,
        "sample": "loop port of the reference algorithm, fp32, query/key rows %d..%d of %d "
                  "(all %d batch*head slabs), time scaled by %d/%d" % (r0, r1 - 1, H, B * N, H, r1 - r0),
        "vectorised_gather_ms": vec_s * 1e3, "c_openmp_ms": c_s * 1e3,
        "host_cpus": cores,
    }


# The benchmark configurations of this operator: name -> (B, heads, side, head_dim, k, dtype);
# `--config NAME` is a shorthand for the matching --batch/--heads/--side/... flags.
CONFIGS = {
    "C1-fp32-check": (1, 2, 16, 32, 3, "fp32"),
    "C2-README-32": (4, 4, 32, 128, 5, "bf16"),
    "C2-README-64": (4, 4, 64, 128, 5, "bf16"),
    "C2-README-128": (4, 4, 128, 128, 5, "bf16"),
    "C2-README-256": (4, 4, 256, 128, 5, "bf16"),
    "C3-fp32-64": (4, 4, 64, 128, 5, "fp32"),
    "C3-fp32-128": (4, 4, 128, 128, 5, "fp32"),
    "C4-k13": (2, 8, 128, 64, 13, "bf16"),
    "C5-stage1": (8, 2, 112, 32, 7, "bf16"),
    "C5-stage2": (8, 4, 56, 32, 7, "bf16"),
    "C5-stage3": (8, 8, 28, 32, 7, "bf16"),
    "C5-stage4": (8, 16, 14, 32, 7, "bf16"),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--side", type=int, default=128)
    ap.add_argument("--batch", type=int, default=4)
    ap.add_argument("--heads", type=int, default=4)
    ap.add_argument("--head-dim", type=int, default=128)
    ap.add_argument("--kernel-size", type=int, default=5)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp16", "fp32"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-sweep", action="store_true", help="skip the other image sides")
    ap.add_argument("--no-unfused", action="store_true",
                    help="skip the unfused qk -> softmax -> av comparator on the GPU")
    ap.add_argument("--simt", action="store_true", help="force the vector-ALU kernels")
    ap.add_argument("--fused-bwd", action="store_true",
                    help="force the fused backward kernel wherever it is built")
    ap.add_argument("--split-bwd", action="store_true",
                    help="force the two-pass backward (dQ, then dK/dV)")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one forward+backward into a HIP graph (torch.cuda.CUDAGraph) "
                         "and time its replays: the step without the host's enqueue cost")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run a plain 256 MiB device copy (calibrates rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--seq", type=int, default=0,
                    help="time natten1d on [batch, heads, SEQ, head_dim] sequences instead of "
                         "natten2d on images (no sweep, no unfused comparator, no CPU baseline)")
    ap.add_argument("--spin-up-ms", type=float, default=60.0,
                    help="untimed steps of the same workload for this long before the warm-up steps: "
                         "from idle the GPU needs ~20 ms of load to settle (steps take 190, then "
                         "200-218, then 182 us at the default shape)")
    ap.add_argument("--event-period", type=int, default=0,
                    help="bracket every N-th launch of each kernel with HIP events (default: steps // 10)")
    ap.add_argument("--config", choices=sorted(CONFIGS),
                    help="one of the named benchmark configurations (sets the shape flags)")
    args = ap.parse_args()
    if args.config:
        (args.batch, args.heads, args.side, args.head_dim, args.kernel_size,
         args.dtype) = CONFIGS[args.config]
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this operator is measured on one GPU only (--gpus 1); "
                 "it has no cross-GPU path, batch*head slabs are independent")

    import torch
    from e_natten_amd import _lib, kernel_path, natten1d, natten2d
    from e_natten_amd import build
    if args.seq:
        args.no_sweep = args.no_unfused = args.no_cpu = True
    if not (os.path.exists(_lib.LIB_PATH) and os.path.exists(build.TORCH_LIB)):
        build.build()
    lib = _lib.load()
    if args.simt:
        lib.enatten_set_path(_lib.PATH_SIMT)
    elif args.fused_bwd:
        lib.enatten_set_path(_lib.PATH_MFMA_FUSED)
    elif args.split_bwd:
        lib.enatten_set_path(_lib.PATH_MFMA_SPLIT)
    dtype = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}[args.dtype]
    B, N, S, D, ks = args.batch, args.heads, args.side, args.head_dim, args.kernel_size
    shape = (B, N, args.seq, D) if args.seq else (B, N, S, S, D)
    op = natten1d if args.seq else natten2d
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    sets, cold = rotating_sets(shape, dtype, dev, 4)
    for st in sets:
        for t in st[:3]:
            t.requires_grad_(True)
    q, k, v, d_o = sets[0]

    def step(i=0):
        q, k, v, d_o = sets[i % len(sets)]
        o = op(q, k, v, ks)
        return torch.autograd.grad(o, (q, k, v), d_o)

    step(0)   # (the first call loads code objects and queries occupancies: not part of the spin-up)
    torch.cuda.synchronize()
    spin_steps = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < args.spin_up_ms:
        for i in range(32):
            step(spin_steps + i)
        torch.cuda.synchronize()
        spin_steps += 32
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    # Per-kernel HIP events inside the timed region: every `period`-th launch of
    # each kernel is bracketed (a record costs ~5 us of queue time; timing all of
    # them would stretch the step by ~7%).
    period = args.event_period if args.event_period > 0 else max(1, args.steps // 10)
    lib.enatten_profile_enable(period)
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    host_s = time.perf_counter() - t0  # time to enqueue all steps
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.enatten_profile_enable(0)
    # the same steps on one set of inputs (whatever fits the caches stays there)
    for _ in range(min(5, args.warmup)):
        step(0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(0)
    torch.cuda.synchronize()
    hot_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    graph_ms = None
    if args.graph:
        # One step recorded on a side stream into a graph, as a caller with a fixed shape
        # would (the library allocates nothing and records no memset; torch's allocator
        # serves the outputs from the graph's private pool), then replayed.
        gq, gk, gv, gd = sets[0]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                torch.autograd.grad(op(gq, gk, gv, ks), (gq, gk, gv), gd)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        cg = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cg):
            g_out = torch.autograd.grad(op(gq, gk, gv, ks), (gq, gk, gv), gd)
        eager = step(0)
        for _ in range(5):
            cg.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a_, b_) for a_, b_ in zip(g_out, eager)), "graph replay differs from eager"
        t0 = time.perf_counter()
        for _ in range(args.steps):
            cg.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        del cg, g_out

    if args.copy_calib:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms_step = elapsed * 1e3 / args.steps
    queries = B * N * (args.seq if args.seq else S * S)
    window = ks if args.seq else ks * ks
    useful = 14.0 * window * D * queries
    alg = (algorithmic_bytes(B, N, 1, args.seq, D, q.element_size()) if args.seq
           else algorithmic_bytes(B, N, S, S, D, q.element_size()))

    kern = {}
    for i, name in enumerate(KERNELS):
        n, tot = ctypes.c_int(), ctypes.c_double()
        lib.enatten_profile_read(i, ctypes.byref(n), ctypes.byref(tot))
        if n.value == 0:
            continue
        empty = ctypes.c_double()
        lib.enatten_profile_read_overhead(i, ctypes.byref(empty))
        raw_us, empty_us = tot.value / n.value * 1e3, empty.value / n.value * 1e3
        # avg_us: the bracket's reading less what the bracket itself adds (an event recorded
        # straight after the closing one, nothing in between, measures that on the same
        # busy queue).  Uncorrected, the brackets of one step sum to more than its wall time.
        kern[name] = {"kernel": lib.enatten_profile_kernel_name(i).decode(), "launches": n.value,
                      "avg_us": raw_us - empty_us, "bracket_us": raw_us, "empty_bracket_us": empty_us,
                      "alg_bytes": alg.get(name, 0)}
    for k in kern.values():
        k["GBps"] = k["alg_bytes"] / (k["avg_us"] * 1e-6) / 1e9
    names = list(kern)
    dom = max(names, key=lambda n: kern[n]["avg_us"])
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if os.path.exists(tpath):
        # counter figures of this very workload, where a profile of it has been taken
        rec = json.load(open(tpath)).get("%s/B%d_N%d_Q%d_d%d_k%d_e%d" % (
            kern[dom]["kernel"], B, N, queries // (B * N), D, window, q.element_size()))
        traffic = rec["bytes_per_launch"] if rec else None
    kernel_ms = sum(kern[n]["avg_us"] for n in names) / 1e3
    roofline = {
        "bound": "hbm", "kernel": kern[dom]["kernel"], "achieved": kern[dom]["GBps"],
        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": kern[dom]["GBps"] / HBM_PEAK_GBS,
        "traffic": traffic,
        "traffic_source": ("profiles/hbm_traffic.txt: rocprofv3 FETCH_SIZE + WRITE_SIZE of an earlier run "
                           "of this workload, not counted in this run") if traffic else None,
        "kernels": kern,
        "path_alg_bytes": alg["path"], "path_kernel_ms": kernel_ms,
        "path_GBps": alg["path"] / (kernel_ms * 1e-3) / 1e9,
        "path_frac": alg["path"] / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
    }
    path = kernel_path(D, ks, dtype)
    if args.seq:   # the 1D matrix-core kernels: bf16 / f16, head dims that are multiples of 8 up to 128, kernel_size <= 49
        path = "mfma" if path != "none" and args.dtype != "fp32" and D % 8 == 0 and 8 <= D <= 128 and 3 <= ks <= 49 \
            else "simt"
    if path == "mfma" and args.dtype in MFMA_PEAK_TF and not args.simt:
        # useful FLOPs against the matrix-core peak of the dtype the kernels compute in
        roofline["mfma_frac_useful"] = useful / (kernel_ms * 1e-3) / 1e12 / MFMA_PEAK_TF[args.dtype]
    working_set = 8 * queries * D * q.element_size()   # q, k, v, o, dO, dq, dk, dv
    out = {
        "metric": "%s fwd+bwd useful TFLOP/s (B%d H%d d%d k%d %s)"
                  % ("natten1d" if args.seq else "natten2d", B, N, D, ks, args.dtype),
        "value": useful / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "spin_up": "%d untimed steps (%.0f ms) before the warm-up steps, so that the timed steps see "
                   "the GPU's settled clocks" % (spin_steps, args.spin_up_ms),
        "timing": "cold: %d input sets in rotation (%s twice the 256 MB memory-side cache)"
                  % (len(sets), "more than" if cold else "LESS than"),
        "hot_ms_per_step": hot_ms,
        "working_set_fits_memory_side_cache": working_set <= MALL_BYTES,
        "host_enqueue_ms_per_step": host_s * 1e3 / args.steps,
        "graph_replay_ms_per_step": graph_ms,
        "kernel_event_sampling": "every %d-th launch; avg_us = bracket_us - empty_bracket_us "
                                 "(an event pair with nothing between, recorded after each bracket)" % period,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": ("natten1d fwd+bwd B=%d heads=%d T=%d head_dim=%d kernel_size=%d"
                                % (B, N, args.seq, D, ks)) if args.seq else
                               ("natten2d fwd+bwd B=%d heads=%d H=W=%d head_dim=%d kernel_size=%d"
                                % (B, N, S, D, ks)),
                   "kernel_path": "simt" if args.simt else path, "queries": queries,
                   "useful_gflop": useful / 1e9},
        "roofline": roofline,
    }
    if not args.no_sweep:
        # The image sides of the reference's benchmark sweeps (bench.py:9 there: forward
        # only, under no_grad, sides 16..512; bench.py:34: forward+backward, sides
        # 16..256), wall-clock only, a few steps each.
        def wall_ms(fn, iters=20):
            for i in range(5):
                fn(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(iters):
                fn(i)
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / iters

        del sets
        torch.cuda.empty_cache()
        sweep = []
        esize = q.element_size()
        for side in (16, 32, 64, 128, 256, 512):
            shp = (B, N, side, side, D)
            ssets, scold = rotating_sets(shp, dtype, dev, 4 if side <= 256 else 3, seed=side)
            qn = B * N * side * side
            with torch.no_grad():
                fwd_ms = wall_ms(lambda i: natten2d(*ssets[i % len(ssets)][:3], ks))
                fwd_hot = wall_ms(lambda i: natten2d(*ssets[0][:3], ks))
            rec = {"side": side, "fwd_ms": fwd_ms, "fwd_hot_ms": fwd_hot,
                   "input_sets": len(ssets), "cold": scold,
                   "fwd_working_set_fits_memory_side_cache": 4 * qn * D * esize <= MALL_BYTES,
                   "fwd_frac_of_hbm_peak": (4 * qn * D * esize + 4 * qn)
                   / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
            if side <= 256 and side != S:
                for st in ssets:
                    for t in st[:3]:
                        t.requires_grad_(True)

                def fb(i, rotate=True):
                    qs, ks_, vs, gs = ssets[i % len(ssets) if rotate else 0]
                    return torch.autograd.grad(natten2d(qs, ks_, vs, ks), (qs, ks_, vs), gs)
                ms = wall_ms(fb)
                ms_hot = wall_ms(lambda i: fb(i, False))
                fl = 14.0 * ks * ks * D * qn
                by = 11 * qn * D * esize + 8 * qn
                rec.update({"ms_per_step": ms, "hot_ms_per_step": ms_hot,
                            "working_set_fits_memory_side_cache": 8 * qn * D * esize <= MALL_BYTES,
                            "useful_tflops": fl / ms / 1e9,
                            "path_frac_of_hbm_peak": by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS})
            sweep.append(rec)
            del ssets
            torch.cuda.empty_cache()
        out["sweep"] = sweep
    if not args.no_unfused:
        gq = torch.Generator(device=dev).manual_seed(1)
        uq, uk, uv, ug = (torch.randn(shape, generator=gq, device=dev, dtype=torch.float32).to(dtype)
                          for _ in range(4))
        try:
            out["unfused_gpu"] = unfused_gpu(uq, uk, uv, ug, ks)
            out["unfused_gpu"]["speedup_fwd_bwd"] = out["unfused_gpu"]["ms_per_step"] / ms_step
        except torch.cuda.OutOfMemoryError as e:
            out["unfused_gpu"] = {"error": "out of memory: %s" % str(e)[:80]}
        del uq, uk, uv, ug
        torch.cuda.empty_cache()
    if not args.no_cpu:
        cb = cpu_baseline(shape, ks, dtype, useful)
        # against the loop port (the headline baseline) and, the conservative figures,
        # against the vectorised torch oracle and the C/OpenMP oracle on all host threads
        cb["gpu_speedup"] = cb["ms"] / ms_step
        cb["gpu_speedup_vs_vectorised_gather"] = cb["vectorised_gather_ms"] / ms_step
        cb["gpu_speedup_vs_c_openmp"] = cb["c_openmp_ms"] / ms_step
        row32 = [r for r in out.get("sweep", []) if r["side"] == 32 and "ms_per_step" in r]
        if cb["loop_port_whole_config"] and row32 and not args.seq:
            cb["loop_port_whole_config"]["gpu_ms"] = row32[0]["ms_per_step"]
            cb["loop_port_whole_config"]["gpu_speedup"] = cb["loop_port_whole_config"]["ms"] / row32[0]["ms_per_step"]
        out["cpu_baseline"] = cb
    print(json.dumps(out))


if __name__ == "__main__":
    main()
