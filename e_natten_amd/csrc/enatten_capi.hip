// C ABI of libenatten.so: argument validation and dispatch.  See enatten.h.

#include <stdarg.h>
#include <stdio.h>

#include <atomic>

#include "na2d_common.h"

namespace enatten {

static thread_local char g_err[512] = "";
static std::atomic<int> g_path{0};

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

namespace {

int elem_size(int dtype) {
    switch (dtype) {
        case ENATTEN_F64: return 8;
        case ENATTEN_F32: return 4;
        case ENATTEN_BF16:
        case ENATTEN_F16: return 2;
    }
    return 0;
}

int check_shape(const char *fn, int B, int N, int H, int W, int D, int ks, int dtype) {
    if (elem_size(dtype) == 0) {
        set_error("%s: unknown dtype code %d (expected ENATTEN_F32/BF16/F16/F64)", fn, dtype);
        return ENATTEN_EINVAL;
    }
    if (B < 1 || N < 1 || H < 1 || W < 1 || D < 1) {
        set_error("%s: every dimension must be >= 1, got B=%d heads=%d H=%d W=%d D=%d", fn, B, N,
                  H, W, D);
        return ENATTEN_EINVAL;
    }
    if (ks < 1 || ks % 2 == 0) {
        set_error("%s: kernel_size must be odd and >= 1, got %d", fn, ks);
        return ENATTEN_EINVAL;
    }
    if (H < ks || W < ks) {
        set_error("%s: image %dx%d is smaller than kernel_size %d", fn, H, W, ks);
        return ENATTEN_EINVAL;
    }
    // elements of one tensor, checked factor by factor so that nothing overflows
    const int64_t limit = (int64_t)1 << 40;
    int64_t count = 1;
    for (const int f : {B, N, H, W, D}) {
        if (count > limit / f) {
            set_error("%s: tensor too large (more than 2^40 elements)", fn);
            return ENATTEN_EUNSUPPORTED;
        }
        count *= f;
    }
    return ENATTEN_OK;
}

int make_view(const char *fn, const char *name, const void *p, const int64_t *st, int N, int H,
              int W, int D, View *out) {
    if (!p) {
        set_error("%s: %s is NULL", fn, name);
        return ENATTEN_EINVAL;
    }
    out->ptr = p;
    if (st) {
        out->sb = st[0]; out->sn = st[1]; out->sh = st[2]; out->sw = st[3];
        if (out->sb < 0 || out->sn < 0 || out->sh < 0 || out->sw < 0) {
            set_error("%s: negative stride for %s", fn, name);
            return ENATTEN_EINVAL;
        }
    } else {
        out->sw = D;
        out->sh = (int64_t)W * D;
        out->sn = (int64_t)H * W * D;
        out->sb = (int64_t)N * H * W * D;
    }
    return ENATTEN_OK;
}

bool use_mfma(int D, int ks, int dtype) {
    return g_path.load() != ENATTEN_PATH_SIMT && mfma_supported(D, ks, dtype);
}
bool use_mfma_f32(int D, int ks, int dtype) {
    return g_path.load() != ENATTEN_PATH_SIMT && mfma_f32_supported(D, ks, dtype);
}
// float32 per query of backward workspace: two for the general and the 16-bit kernels
// (delta and 1/Z), 2 * ks * ks for the float32 matrix-core kernels (P and dS), four for
// float64 tensors (two doubles: the log-sum-exp in double and delta)
size_t ws_floats_per_query(int D, int ks, int dtype) {
    if (dtype == ENATTEN_F64) return 4;
    return mfma_f32_supported(D, ks, dtype) ? mfma_f32_workspace_floats(ks) : 2;
}
// Layout of dq, dk, dv: contiguous [B, heads, H, W, D], or the caller's element strides on
// (batch, head, row, column) with unit stride on the channels.  Call after a->s is set.
int set_grad_layout(const char *fn, BwdArgs *a, const int64_t *st) {
    const Shape &s = a->s;
    if (st) {
        a->gsb = st[0]; a->gsn = st[1]; a->gsh = st[2]; a->gsw = st[3];
        if (a->gsb < 0 || a->gsn < 0 || a->gsh < 0 || a->gsw < s.D) {
            set_error("%s: gradient strides must be non-negative, and at least D between pixels", fn);
            return ENATTEN_EINVAL;
        }
    } else {
        a->gsw = s.D;
        a->gsh = (int64_t)s.W * s.D;
        a->gsn = (int64_t)s.H * s.W * s.D;
        a->gsb = (int64_t)s.N * s.H * s.W * s.D;
    }
    return ENATTEN_OK;
}
// float64 tensors: one kernel family (na2d_f64.hip), whatever the path setting
int bwd_f64(const char *fn, const BwdArgs &a, size_t ws_floats, hipStream_t st) {
    if (ws_floats < (size_t)4 * a.s.B * a.s.N * a.s.H * a.s.W) {
        set_error("%s: float64 tensors need 16 bytes of workspace per query", fn);
        return ENATTEN_EUNSUPPORTED;
    }
    return launch_bwd_f64(a, st);
}

}  // namespace
}  // namespace enatten

using namespace enatten;

extern "C" {
#pragma GCC visibility push(default)

int enatten_abi_version(void) { return ENATTEN_ABI_VERSION; }

const char *enatten_last_error(void) { return g_err; }

int enatten2d_kernel_path(int D, int kernel_size, int dtype) {
    if (elem_size(dtype) == 0 || D < 1 || D > 1024 || kernel_size < 1 || kernel_size % 2 == 0)
        return ENATTEN_PATH_NONE;
    return use_mfma(D, kernel_size, dtype) || use_mfma_f32(D, kernel_size, dtype) ? ENATTEN_PATH_MFMA
                                                                                  : ENATTEN_PATH_SIMT;
}

int enatten_set_path(int path) {
    if (path != 0 && path != ENATTEN_PATH_SIMT && path != ENATTEN_PATH_MFMA_FUSED &&
        path != ENATTEN_PATH_MFMA_SPLIT && path != ENATTEN_PATH_MFMA_SPLIT_QUEUE)
        return g_path.load();
    return g_path.exchange(path);
}

int enatten2d_fwd(const void *q, const void *k, const void *v, void *o, float *lse, int B,
                  int heads, int H, int W, int D, int kernel_size, int dtype,
                  const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                  const int64_t *o_strides, float scale, void *stream) {
    const char *fn = "enatten2d_fwd";
    int rc = check_shape(fn, B, heads, H, W, D, kernel_size, dtype);
    if (rc) return rc;
    FwdArgs a;
    if ((rc = make_view(fn, "q", q, q_strides, heads, H, W, D, &a.q))) return rc;
    if ((rc = make_view(fn, "k", k, k_strides, heads, H, W, D, &a.k))) return rc;
    if ((rc = make_view(fn, "v", v, v_strides, heads, H, W, D, &a.v))) return rc;
    if ((rc = make_view(fn, "o", o, o_strides, heads, H, W, D, &a.o))) return rc;
    a.lse = lse;
    a.s = Shape{B, heads, H, W, D, kernel_size, kernel_size, scale};
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ENATTEN_F64) return launch_fwd_f64(a, st);
    if (use_mfma(D, kernel_size, dtype)) return launch_fwd_mfma(a, dtype, st);
    if (use_mfma_f32(D, kernel_size, dtype)) return launch_fwd_mfma_f32(a, st);
    return launch_fwd_simt(a, dtype, st);
}

size_t enatten2d_bwd_workspace_bytes(int B, int heads, int H, int W, int D, int kernel_size,
                                     int dtype) {
    if (B < 1 || heads < 1 || H < 1 || W < 1 || D < 1 || kernel_size < 1) return 0;
    return (size_t)B * heads * H * W * ws_floats_per_query(D, kernel_size, dtype) * sizeof(float);
}

// Shared body of the two backward entry points: `workspace` holds two float32 per query.
static int bwd2d(const char *fn, const void *q, const void *k, const void *v, const void *o,
                 const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                 float *workspace, size_t ws_floats, int B, int heads, int H, int W, int D, int kernel_size,
                 int dtype, const int64_t *q_strides, const int64_t *k_strides,
                 const int64_t *v_strides, const int64_t *o_strides, const int64_t *do_strides,
                 float scale, void *stream, const int64_t *grad_strides = nullptr) {
    BwdArgs a;
    int rc;
    if ((rc = make_view(fn, "q", q, q_strides, heads, H, W, D, &a.q))) return rc;
    if ((rc = make_view(fn, "k", k, k_strides, heads, H, W, D, &a.k))) return rc;
    if ((rc = make_view(fn, "v", v, v_strides, heads, H, W, D, &a.v))) return rc;
    if ((rc = make_view(fn, "o", o, o_strides, heads, H, W, D, &a.o))) return rc;
    if ((rc = make_view(fn, "d_o", d_o, do_strides, heads, H, W, D, &a.d_o))) return rc;
    if (!lse || !dq || !dk || !dv) {
        set_error("%s: lse, dq, dk and dv must all be non-NULL", fn);
        return ENATTEN_EINVAL;
    }
    a.lse = lse;
    a.dq = dq; a.dk = dk; a.dv = dv;
    a.delta = workspace;
    a.zinv = a.delta + (size_t)B * heads * H * W;
    a.s = Shape{B, heads, H, W, D, kernel_size, kernel_size, scale};
    if ((rc = set_grad_layout(fn, &a, grad_strides))) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (dtype == ENATTEN_F64) return bwd_f64(fn, a, ws_floats, st);
    if (use_mfma(D, kernel_size, dtype)) return launch_bwd_mfma(a, dtype, g_path.load(), st);
    // the float32 matrix-core backward where the workspace at hand holds its P and dS (it
    // writes contiguous gradients only)
    if (use_mfma_f32(D, kernel_size, dtype) && a.grads_contiguous() &&
        ws_floats >= (size_t)B * heads * H * W * mfma_f32_workspace_floats(kernel_size))
        return launch_bwd_mfma_f32(a, st);
    return launch_bwd_simt(a, dtype, st);
}

int enatten2d_bwd(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                  const float *lse, void *dq, void *dk, void *dv, void *workspace, int B,
                  int heads, int H, int W, int D, int kernel_size, int dtype,
                  const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                  const int64_t *o_strides, const int64_t *do_strides, float scale,
                  void *stream) {
    const char *fn = "enatten2d_bwd";
    const int rc = check_shape(fn, B, heads, H, W, D, kernel_size, dtype);
    if (rc) return rc;
    if (!workspace) {
        set_error("%s: workspace is NULL", fn);
        return ENATTEN_EINVAL;
    }
    // the caller provides enatten2d_bwd_workspace_bytes() for this very call
    return bwd2d(fn, q, k, v, o, d_o, lse, dq, dk, dv, static_cast<float *>(workspace),
                 (size_t)B * heads * H * W * ws_floats_per_query(D, kernel_size, dtype), B, heads,
                 H, W, D, kernel_size, dtype, q_strides, k_strides, v_strides, o_strides,
                 do_strides, scale, stream);
}

int enatten2d_bwd_into(const void *q, const void *k, const void *v, const void *o,
                       const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                       void *workspace, int B, int heads, int H, int W, int D, int kernel_size,
                       int dtype, const int64_t *q_strides, const int64_t *k_strides,
                       const int64_t *v_strides, const int64_t *o_strides,
                       const int64_t *do_strides, const int64_t *grad_strides, float scale,
                       void *stream) {
    const char *fn = "enatten2d_bwd_into";
    const int rc = check_shape(fn, B, heads, H, W, D, kernel_size, dtype);
    if (rc) return rc;
    if (!workspace) {
        set_error("%s: workspace is NULL", fn);
        return ENATTEN_EINVAL;
    }
    return bwd2d(fn, q, k, v, o, d_o, lse, dq, dk, dv, static_cast<float *>(workspace),
                 (size_t)B * heads * H * W * ws_floats_per_query(D, kernel_size, dtype), B, heads,
                 H, W, D, kernel_size, dtype, q_strides, k_strides, v_strides, o_strides,
                 do_strides, scale, stream, grad_strides);
}

// ---- backward without a caller-provided workspace ---------------------------
// The two float32 per query that the backward passes hand to each other live in a
// device array of this library instead.  Every GPU holds its own copy of the array at
// its own address; `scratch` below is only the host-side handle of the symbol, the
// address on the current device comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) float scratch[2 * (size_t)ENATTEN_STATIC_BWD_MAX_QUERIES];

namespace {
constexpr int kMaxDevices = 64;
std::atomic<float *> g_scratch_ptr[kMaxDevices];

int scratch_of_current_device(const char *fn, float **out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("%s: no current HIP device (or a device number beyond %d)", fn, kMaxDevices - 1);
        return ENATTEN_ELAUNCH;
    }
    float *p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // two threads may both ask; they get the same answer
        const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            set_error("%s: hipGetSymbolAddress(scratch) failed: %s", fn, hipGetErrorString(e));
            return ENATTEN_ELAUNCH;
        }
        g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return ENATTEN_OK;
}
}  // namespace

int enatten2d_bwd_static(const void *q, const void *k, const void *v, const void *o,
                         const void *d_o, const float *lse, void *dq, void *dk, void *dv, int B,
                         int heads, int H, int W, int D, int kernel_size, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *do_strides, float scale, void *stream) {
    const char *fn = "enatten2d_bwd_static";
    int rc = check_shape(fn, B, heads, H, W, D, kernel_size, dtype);
    if (rc) return rc;
    if ((int64_t)B * heads * H * W > (int64_t)ENATTEN_STATIC_BWD_MAX_QUERIES) {
        set_error("%s: %lld queries exceed the %d that the built-in scratch holds; use "
                  "enatten2d_bwd with a workspace", fn, (long long)B * heads * H * W,
                  ENATTEN_STATIC_BWD_MAX_QUERIES);
        return ENATTEN_EUNSUPPORTED;
    }
    float *ws = nullptr;
    if ((rc = scratch_of_current_device(fn, &ws))) return rc;
    // Nothing in the scratch has to start at zero: the first pass writes both values of
    // every query before the second pass reads them.
    return bwd2d(fn, q, k, v, o, d_o, lse, dq, dk, dv, ws,
                 (size_t)2 * ENATTEN_STATIC_BWD_MAX_QUERIES, B, heads, H, W, D, kernel_size, dtype,
                 q_strides, k_strides, v_strides, o_strides, do_strides, scale, stream);
}

// ---- rectangular and causal windows ----------------------------------------
// One axis of a window: extent k, causal or centred.
static int check_axis(const char *fn, const char *axis, int L, int k, int causal) {
    if (k < 1 || (!causal && k % 2 == 0)) {
        set_error("%s: kernel_%s must be >= 1, and odd unless that axis is causal, got %d", fn,
                  axis, k);
        return ENATTEN_EINVAL;
    }
    if (L < k) {
        set_error("%s: the image has %d positions along %s, fewer than kernel_%s = %d", fn, L, axis,
                  axis, k);
        return ENATTEN_EINVAL;
    }
    return ENATTEN_OK;
}

int enatten2d_fwd_window(const void *q, const void *k, const void *v, const void *rpb, void *o,
                         float *lse, int B, int heads, int H, int W, int D, int kernel_h,
                         int kernel_w, int causal_h, int causal_w, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides, float scale,
                         void *stream) {
    if (kernel_h == kernel_w && !causal_h && !causal_w && !rpb)
        return enatten2d_fwd(q, k, v, o, lse, B, heads, H, W, D, kernel_h, dtype, q_strides,
                             k_strides, v_strides, o_strides, scale, stream);
    const char *fn = "enatten2d_fwd_window";
    int rc = check_shape(fn, B, heads, H, W, D, 1, dtype);
    if (rc) return rc;
    if ((rc = check_axis(fn, "h", H, kernel_h, causal_h))) return rc;
    if ((rc = check_axis(fn, "w", W, kernel_w, causal_w))) return rc;
    if (rpb && (causal_h || causal_w)) {
        set_error("%s: a relative position bias goes with centred axes only", fn);
        return ENATTEN_EINVAL;
    }
    FwdArgs a;
    if ((rc = make_view(fn, "q", q, q_strides, heads, H, W, D, &a.q))) return rc;
    if ((rc = make_view(fn, "k", k, k_strides, heads, H, W, D, &a.k))) return rc;
    if ((rc = make_view(fn, "v", v, v_strides, heads, H, W, D, &a.v))) return rc;
    if ((rc = make_view(fn, "o", o, o_strides, heads, H, W, D, &a.o))) return rc;
    a.lse = lse;
    a.s = Shape{B, heads, H, W, D, kernel_h, kernel_w, scale, causal_h ? 1 : 0, causal_w ? 1 : 0};
    a.rpb = rpb;
    if (dtype == ENATTEN_F64) return launch_fwd_f64(a, static_cast<hipStream_t>(stream));
    return launch_fwd_simt(a, dtype, static_cast<hipStream_t>(stream));
}

size_t enatten2d_bwd_window_workspace_bytes(int B, int heads, int H, int W, int kernel_h,
                                            int kernel_w, int with_rpb) {
    if (B < 1 || heads < 1 || H < 1 || W < 1 || kernel_h < 1 || kernel_w < 1) return 0;
    // four floats per query (float64 tensors use all four), and with a bias dS of every
    // (query, window position)
    return (size_t)B * heads * H * W * (4 + (with_rpb ? (size_t)kernel_h * kernel_w : 0)) * sizeof(float);
}

int enatten2d_bwd_window(const void *q, const void *k, const void *v, const void *rpb,
                         const void *o, const void *d_o, const float *lse, void *dq, void *dk,
                         void *dv, float *d_rpb, void *workspace, int B, int heads, int H, int W,
                         int D, int kernel_h, int kernel_w, int causal_h, int causal_w, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *do_strides, float scale, void *stream) {
    const char *fn = "enatten2d_bwd_window";
    const bool plain = kernel_h == kernel_w && !causal_h && !causal_w && !rpb;
    int rc = check_shape(fn, B, heads, H, W, D, plain ? kernel_h : 1, dtype);
    if (rc) return rc;
    if (!workspace) {
        set_error("%s: workspace is NULL", fn);
        return ENATTEN_EINVAL;
    }
    const size_t ws_floats = (size_t)B * heads * H * W * (dtype == ENATTEN_F64 ? 4 : 2);
    if (plain)  // the reference's window: every kernel family that two floats per query allow
        return bwd2d(fn, q, k, v, o, d_o, lse, dq, dk, dv, static_cast<float *>(workspace),
                     ws_floats, B, heads, H, W, D, kernel_h, dtype, q_strides, k_strides, v_strides,
                     o_strides, do_strides, scale, stream);
    if ((rc = check_axis(fn, "h", H, kernel_h, causal_h))) return rc;
    if ((rc = check_axis(fn, "w", W, kernel_w, causal_w))) return rc;
    if (rpb && (causal_h || causal_w)) {
        set_error("%s: a relative position bias goes with centred axes only", fn);
        return ENATTEN_EINVAL;
    }
    if (!rpb != !d_rpb) {
        set_error("%s: rpb and d_rpb come together", fn);
        return ENATTEN_EINVAL;
    }
    BwdArgs a;
    if ((rc = make_view(fn, "q", q, q_strides, heads, H, W, D, &a.q))) return rc;
    if ((rc = make_view(fn, "k", k, k_strides, heads, H, W, D, &a.k))) return rc;
    if ((rc = make_view(fn, "v", v, v_strides, heads, H, W, D, &a.v))) return rc;
    if ((rc = make_view(fn, "o", o, o_strides, heads, H, W, D, &a.o))) return rc;
    if ((rc = make_view(fn, "d_o", d_o, do_strides, heads, H, W, D, &a.d_o))) return rc;
    if (!lse || !dq || !dk || !dv) {
        set_error("%s: lse, dq, dk and dv must all be non-NULL", fn);
        return ENATTEN_EINVAL;
    }
    a.lse = lse;
    a.dq = dq; a.dk = dk; a.dv = dv;
    a.delta = static_cast<float *>(workspace);
    a.zinv = a.delta + (size_t)B * heads * H * W;
    a.s = Shape{B, heads, H, W, D, kernel_h, kernel_w, scale, causal_h ? 1 : 0, causal_w ? 1 : 0};
    if ((rc = set_grad_layout(fn, &a, nullptr))) return rc;
    a.rpb = rpb;
    a.d_rpb = d_rpb;
    a.ds_pairs = rpb ? a.delta + (size_t)4 * B * heads * H * W : nullptr;
    if (dtype == ENATTEN_F64) return bwd_f64(fn, a, ws_floats, static_cast<hipStream_t>(stream));
    return launch_bwd_simt(a, dtype, static_cast<hipStream_t>(stream));
}

static int view_1d(const char *fn, const char *name, const void *p, const int64_t *st, int N,
                   int T, int D, View *out) {
    if (!p) {
        set_error("%s: %s is NULL", fn, name);
        return ENATTEN_EINVAL;
    }
    out->ptr = p;
    out->sh = 0;
    if (st) {
        out->sb = st[0]; out->sn = st[1]; out->sw = st[2];
        if (out->sb < 0 || out->sn < 0 || out->sw < 0) {
            set_error("%s: negative stride for %s", fn, name);
            return ENATTEN_EINVAL;
        }
    } else {
        out->sw = D;
        out->sn = (int64_t)T * D;
        out->sb = (int64_t)N * T * D;
    }
    return ENATTEN_OK;
}

// A sequence is a 1 x T image with a 1 x k window: the size limit applies to
// B * heads * T * D elements.
static int check_shape_1d(const char *fn, int B, int N, int T, int D, int ks, int dtype) {
    if (ks >= 1 && ks % 2 == 1 && T >= 1 && T < ks) {
        set_error("%s: sequence length %d is smaller than kernel_size %d", fn, T, ks);
        return ENATTEN_EINVAL;
    }
    if (ks < 1 || ks % 2 == 0) return check_shape(fn, B, N, 1, T, D, ks, dtype);  // reports it
    return check_shape(fn, B, N, 1, T, D, 1, dtype);
}

int enatten1d_fwd(const void *q, const void *k, const void *v, void *o, float *lse, int B,
                  int heads, int T, int D, int kernel_size, int dtype, const int64_t *q_strides,
                  const int64_t *k_strides, const int64_t *v_strides, const int64_t *o_strides,
                  float scale, void *stream) {
    const char *fn = "enatten1d_fwd";
    int rc = check_shape_1d(fn, B, heads, T, D, kernel_size, dtype);
    if (rc) return rc;
    FwdArgs a;
    if ((rc = view_1d(fn, "q", q, q_strides, heads, T, D, &a.q))) return rc;
    if ((rc = view_1d(fn, "k", k, k_strides, heads, T, D, &a.k))) return rc;
    if ((rc = view_1d(fn, "v", v, v_strides, heads, T, D, &a.v))) return rc;
    if ((rc = view_1d(fn, "o", o, o_strides, heads, T, D, &a.o))) return rc;
    a.lse = lse;
    a.s = Shape{B, heads, 1, T, D, 1, kernel_size, scale};  // a 1 x k window on a 1 x T image
    if (dtype == ENATTEN_F64) return launch_fwd_f64(a, static_cast<hipStream_t>(stream));
    if (g_path.load() != ENATTEN_PATH_SIMT && mfma1d_supported(D, kernel_size, dtype))
        return launch_fwd1d_mfma(a, dtype, static_cast<hipStream_t>(stream));
    return launch_fwd_simt(a, dtype, static_cast<hipStream_t>(stream));
}

size_t enatten1d_bwd_workspace_bytes(int B, int heads, int T) {
    if (B < 1 || heads < 1 || T < 1) return 0;
    return (size_t)B * heads * T * 4 * sizeof(float);  // float64 tensors use all four
}

int enatten1d_bwd(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                  const float *lse, void *dq, void *dk, void *dv, void *workspace, int B,
                  int heads, int T, int D, int kernel_size, int dtype, const int64_t *q_strides,
                  const int64_t *k_strides, const int64_t *v_strides, const int64_t *o_strides,
                  const int64_t *do_strides, float scale, void *stream) {
    return enatten1d_bwd_into(q, k, v, o, d_o, lse, dq, dk, dv, workspace, B, heads, T, D, kernel_size,
                              dtype, q_strides, k_strides, v_strides, o_strides, do_strides, nullptr,
                              scale, stream);
}

int enatten1d_bwd_into(const void *q, const void *k, const void *v, const void *o, const void *d_o,
                       const float *lse, void *dq, void *dk, void *dv, void *workspace, int B,
                       int heads, int T, int D, int kernel_size, int dtype,
                       const int64_t *q_strides, const int64_t *k_strides, const int64_t *v_strides,
                       const int64_t *o_strides, const int64_t *do_strides,
                       const int64_t *grad_strides, float scale, void *stream) {
    const char *fn = grad_strides ? "enatten1d_bwd_into" : "enatten1d_bwd";
    int rc = check_shape_1d(fn, B, heads, T, D, kernel_size, dtype);
    if (rc) return rc;
    BwdArgs a;
    if ((rc = view_1d(fn, "q", q, q_strides, heads, T, D, &a.q))) return rc;
    if ((rc = view_1d(fn, "k", k, k_strides, heads, T, D, &a.k))) return rc;
    if ((rc = view_1d(fn, "v", v, v_strides, heads, T, D, &a.v))) return rc;
    if ((rc = view_1d(fn, "o", o, o_strides, heads, T, D, &a.o))) return rc;
    if ((rc = view_1d(fn, "d_o", d_o, do_strides, heads, T, D, &a.d_o))) return rc;
    if (!lse || !dq || !dk || !dv || !workspace) {
        set_error("%s: lse, dq, dk, dv and workspace must all be non-NULL", fn);
        return ENATTEN_EINVAL;
    }
    a.lse = lse;
    a.dq = dq; a.dk = dk; a.dv = dv;
    a.delta = static_cast<float *>(workspace);
    a.zinv = a.delta + (size_t)B * heads * T;
    a.s = Shape{B, heads, 1, T, D, 1, kernel_size, scale};
    {
        // (batch, head, position) strides -> the four of an image with one row
        const int64_t g4[4] = {grad_strides ? grad_strides[0] : 0, grad_strides ? grad_strides[1] : 0, 0,
                               grad_strides ? grad_strides[2] : 0};
        if ((rc = set_grad_layout(fn, &a, grad_strides ? g4 : nullptr))) return rc;
    }
    if (dtype == ENATTEN_F64)
        return bwd_f64(fn, a, (size_t)4 * B * heads * T, static_cast<hipStream_t>(stream));
    if (g_path.load() != ENATTEN_PATH_SIMT && mfma1d_supported(D, kernel_size, dtype))
        return launch_bwd1d_mfma(a, dtype, g_path.load(), static_cast<hipStream_t>(stream));
    return launch_bwd_simt(a, dtype, static_cast<hipStream_t>(stream));
}

#pragma GCC visibility pop
}  // extern "C"
