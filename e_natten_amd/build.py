"""Compile the HIP sources in csrc/ into e_natten_amd/libenatten.so for gfx950,
and the native torch binding csrc/torch_shim.cpp into libenatten_torch.so.

Run as ``python -m e_natten_amd.build``.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libenatten.so")
TORCH_LIB = os.path.join(HERE, "libenatten_torch.so")
SOURCES = ["na2d_mfma.hip", "na2d_mfma_narrow.hip", "enatten_capi.hip", "enatten_prof.cpp", "na2d_simt.hip",
           "na2d_f64.hip", "na2d_mfma_fused.hip", "na2d_mfma_onepass.hip", "na2d_mfma_f32.hip", "na1d_mfma.hip", "na1d_mfma_narrow.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


# Per-source additions.  The fused backward is bound by instruction latency at two waves
# per SIMD; the scheduler strategy that favours instruction-level parallelism keeps more
# LDS reads in flight ahead of the matrix instructions there (measured 156 -> 147 us at
# B4 N4 128x128, d=128, k=5).  The other kernels were measured slower or equal with it.
EXTRA_FLAGS = {"na2d_mfma_fused.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]}


def _hipcc() -> str:
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def _up_to_date(src: str, obj: str) -> bool:
    if not os.path.exists(obj):
        return False
    deps = [os.path.join(CSRC, src), os.path.join(ROOT, "include", "enatten.h")]
    deps += [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    return all(os.path.getmtime(d) <= os.path.getmtime(obj) for d in deps)


def _compile(src: str, incremental: bool = False) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    if incremental and _up_to_date(src, obj):
        return obj
    cmd = [_hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr[-4000:]))
    return obj


def _build_torch_shim() -> str:
    """Host-only C++ against the headers of the installed torch; links libenatten.so
    (found beside it at run time) and the torch libraries the process has loaded."""
    import torch
    from torch.utils import cpp_extension
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch.compiled_with_cxx11_abi()),
           "-I", os.path.join(ROOT, "include")]
    for inc in cpp_extension.include_paths():
        cmd += ["-isystem", inc]
    cmd += ["-isystem", "/opt/rocm/include", os.path.join(CSRC, "torch_shim.cpp"), "-o", TORCH_LIB,
            "-L", HERE, "-lenatten", "-L", tlib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
            "-Wl,-rpath,$ORIGIN", "-Wl,--no-as-needed"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the torch binding failed:\n%s" % r.stderr[-4000:])
    return TORCH_LIB


def build(verbose: bool = False, incremental: bool = False) -> str:
    """Compile every source (with `incremental`, only those older than their object
    file's inputs) and link libenatten.so and the torch binding; returns the path of
    libenatten.so."""
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as ex:
        objs = list(ex.map(lambda src: _compile(src, incremental), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s" % r.stderr[-4000:])
    shim_deps = [os.path.join(CSRC, "torch_shim.cpp"), os.path.join(ROOT, "include", "enatten.h")]
    if not (incremental and os.path.exists(TORCH_LIB) and
            all(os.path.getmtime(d) <= os.path.getmtime(TORCH_LIB) for d in shim_deps)):
        _build_torch_shim()
    if verbose:
        print("built", LIB, "and", TORCH_LIB)
    return LIB


if __name__ == "__main__":
    build(verbose=True, incremental="--incremental" in sys.argv[1:])
    sys.exit(0)
