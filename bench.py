"""Benchmark of the fused 2D neighborhood attention hot path on one MI355X.

A step is one forward + backward of ``natten2d`` (through the autograd Function
and the C ABI) on the reference's benchmark shape (bench.py:14,39 of the
reference: B=4, heads=4, head_dim=128, kernel_size=5) in bf16 at image side 128.
Prints ONE JSON line.  `value` is useful TFLOP/s (14*k^2*d FLOP per query);
`roofline` is the achieved algorithmic HBM bandwidth of the slowest kernel, from
HIP events recorded around every kernel launch inside the timed region;
`cpu_baseline` times the CPU restatement of the reference's algorithm on this
machine's host cores on a bounded sample of the same workload.
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
MFMA_BF16_PEAK_TF = 2500.0   # dense bf16, published
KERNELS = ("fwd", "bwd_dq", "bwd_dkdv", "bwd_fused")


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
    return {
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
    ap.add_argument("--simt", action="store_true", help="force the vector-ALU kernels")
    ap.add_argument("--fused-bwd", action="store_true",
                    help="force the fused backward kernel wherever it is built")
    ap.add_argument("--split-bwd", action="store_true",
                    help="force the two-pass backward (dQ, then dK/dV)")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run a plain 256 MiB device copy (calibrates rocprofv3 "
                         "FETCH_SIZE / WRITE_SIZE readings)")
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
    from e_natten_amd import _lib, kernel_path, natten2d
    from e_natten_amd import build
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
    shape = (B, N, S, S, D)
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    q, k, v, d_o = (torch.randn(shape, generator=g).to(dtype).to(dev) for _ in range(4))
    q.requires_grad_(True); k.requires_grad_(True); v.requires_grad_(True)

    def step():
        o = natten2d(q, k, v, ks)
        return torch.autograd.grad(o, (q, k, v), d_o)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # Per-kernel HIP events inside the timed region: every `period`-th launch of
    # each kernel is bracketed (a record costs ~3 us of queue time; timing all of
    # them would stretch the step by ~10%).
    period = max(1, args.steps // 10)
    lib.enatten_profile_enable(period)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    host_s = time.perf_counter() - t0  # time to enqueue all steps
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.enatten_profile_enable(0)

    if args.copy_calib:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms_step = elapsed * 1e3 / args.steps
    queries = B * N * S * S
    useful = 14.0 * ks * ks * D * queries
    alg = algorithmic_bytes(B, N, S, S, D, q.element_size())

    kern = {}
    for i, name in enumerate(KERNELS):
        n, tot = ctypes.c_int(), ctypes.c_double()
        lib.enatten_profile_read(i, ctypes.byref(n), ctypes.byref(tot))
        if n.value == 0:
            continue
        avg_ms = tot.value / n.value
        kern[name] = {"kernel": lib.enatten_profile_kernel_name(i).decode(), "launches": n.value,
                      "avg_us": avg_ms * 1e3, "alg_bytes": alg.get(name, 0)}
    for k in kern.values():
        k["GBps"] = k["alg_bytes"] / (k["avg_us"] * 1e-6) / 1e9
    names = list(kern)
    dom = max(names, key=lambda n: kern[n]["avg_us"])
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.txt")
    if os.path.exists(tpath):
        rec = json.load(open(tpath)).get("%s/side%d/%s" % (kern[dom]["kernel"], S, args.dtype))
        traffic = rec["bytes_per_launch"] if rec else None
    kernel_ms = sum(kern[n]["avg_us"] for n in names) / 1e3
    roofline = {
        "bound": "hbm", "kernel": kern[dom]["kernel"], "achieved": kern[dom]["GBps"],
        "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": kern[dom]["GBps"] / HBM_PEAK_GBS,
        "traffic": traffic, "kernels": kern,
        "path_alg_bytes": alg["path"], "path_kernel_ms": kernel_ms,
        "path_GBps": alg["path"] / (kernel_ms * 1e-3) / 1e9,
        "path_frac": alg["path"] / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "mfma_frac_useful": useful / (kernel_ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TF,
    }
    out = {
        "metric": "natten2d fwd+bwd useful TFLOP/s (B4 H4 d128 k5 bf16)",
        "value": useful / (ms_step * 1e-3) / 1e12, "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "host_enqueue_ms_per_step": host_s * 1e3 / args.steps,
        "kernel_event_sampling": "every %d-th launch" % period,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": "natten2d fwd+bwd B=%d heads=%d H=W=%d head_dim=%d kernel_size=%d"
                               % (B, N, S, D, ks),
                   "kernel_path": kernel_path(D, ks, dtype), "queries": queries,
                   "useful_gflop": useful / 1e9},
        "roofline": roofline,
    }
    if not args.no_sweep:
        # The image sides of the reference's benchmark sweeps (bench.py:9 there: forward
        # only, under no_grad, sides 16..512; bench.py:34: forward+backward, sides
        # 16..256), wall-clock only, a few steps each.
        def wall_ms(fn, iters=20):
            for _ in range(5):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(iters):
                fn()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) * 1e3 / iters

        sweep = []
        for side in (16, 32, 64, 128, 256, 512):
            shp = (B, N, side, side, D)
            qs, ks_, vs = (torch.randn(shp, generator=g).to(dtype).to(dev) for _ in range(3))
            qn = B * N * side * side
            with torch.no_grad():
                fwd_ms = wall_ms(lambda: natten2d(qs, ks_, vs, ks))
            rec = {"side": side, "fwd_ms": fwd_ms,
                   "fwd_frac_of_hbm_peak": (4 * qn * D * qs.element_size() + 4 * qn)
                   / (fwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBS}
            if side <= 256 and side != S:
                gs = torch.randn(shp, generator=g).to(dtype).to(dev)
                for t in (qs, ks_, vs):
                    t.requires_grad_(True)
                ms = wall_ms(lambda: torch.autograd.grad(natten2d(qs, ks_, vs, ks), (qs, ks_, vs), gs))
                fl = 14.0 * ks * ks * D * qn
                by = 11 * qn * D * qs.element_size() + 8 * qn
                rec.update({"ms_per_step": ms, "useful_tflops": fl / ms / 1e9,
                            "path_frac_of_hbm_peak": by / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                            "mfma_frac_useful": fl / ms / 1e9 / MFMA_BF16_PEAK_TF})
                del gs
            sweep.append(rec)
            del qs, ks_, vs
        out["sweep"] = sweep
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(shape, ks, dtype, useful)
        out["cpu_baseline"]["gpu_speedup"] = out["cpu_baseline"]["ms"] / ms_step
    print(json.dumps(out))


if __name__ == "__main__":
    main()
