// General neighborhood-attention kernels on the vector ALUs (fp32 FMA).
//
// They serve every shape the matrix-core kernels do not: float32 tensors (true
// fp32 arithmetic, no reduced-precision products), head dims that are not 32 /
// 64 / 128, and rectangular windows.  Each query (or key, in the dK/dV pass) is
// owned by a group of G adjacent lanes; a lane holds 8 contiguous channels per
// chunk, dot products are finished with xor-shuffles inside the group, and K/V
// rows are read straight from global memory (16-byte loads when the layout
// allows), relying on L1/L2 for the k*k-fold reuse between neighbouring queries.
//
// Math per query follows e_natten/pytorch.py:196-202 (forward) and :248-288
// (backward), with the softmax Jacobian product written as
// dS = P * (dP - sum(P * dP)) and sum(P * dP) obtained as dO . O.

#include <math.h>

#include "na2d_common.h"

namespace enatten {
namespace {

struct bf16_t { uint16_t x; };
struct f16_t { _Float16 x; };

__device__ inline float cvt_in(float v) { return v; }
__device__ inline float cvt_in(bf16_t v) { return __uint_as_float(((uint32_t)v.x) << 16); }
__device__ inline float cvt_in(f16_t v) { return (float)v.x; }

__device__ inline void cvt_out(float f, float &o) { o = f; }
__device__ inline void cvt_out(float f, bf16_t &o) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) { o.x = (uint16_t)((u >> 16) | 0x40); return; }
    u += 0x7fffu + ((u >> 16) & 1u);
    o.x = (uint16_t)(u >> 16);
}
__device__ inline void cvt_out(float f, f16_t &o) { o.x = (_Float16)f; }

// 8 channels starting at p; channels at or past `nvalid` read as zero.
template <typename T, bool VEC>
__device__ inline void load8(const T *p, int nvalid, float (&x)[8]) {
    if (VEC) {
        if (nvalid <= 0) {
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = 0.f;
            return;
        }
        if (sizeof(T) == 4) {
            const float4 a = *reinterpret_cast<const float4 *>(p);
            const float4 b = *reinterpret_cast<const float4 *>(p + 4);
            x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
            x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
        } else {
            union { uint4 u; T t[8]; } r;
            r.u = *reinterpret_cast<const uint4 *>(p);
#pragma unroll
            for (int e = 0; e < 8; e++) x[e] = cvt_in(r.t[e]);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = e < nvalid ? cvt_in(p[e]) : 0.f;
    }
}

template <typename T, bool VEC>
__device__ inline void store8(T *p, int nvalid, const float (&x)[8]) {
    if (nvalid <= 0) return;
    if (VEC) {
        if (sizeof(T) == 4) {
            *reinterpret_cast<float4 *>(p) = make_float4(x[0], x[1], x[2], x[3]);
            *reinterpret_cast<float4 *>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
        } else {
            union { uint4 u; T t[8]; } r;
#pragma unroll
            for (int e = 0; e < 8; e++) cvt_out(x[e], r.t[e]);
            *reinterpret_cast<uint4 *>(p) = r.u;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++)
            if (e < nvalid) cvt_out(x[e], p[e]);
    }
}

template <int G, typename A>
__device__ inline A group_sum(A x) {
#pragma unroll
    for (int off = G / 2; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

// Accumulator of the q.k logits.  With float32 tensors and unscaled logits of
// magnitude ~50 a float32 dot product is only good to ~1e-5, which the
// exponential turns into a 1e-5 relative error of P and ~1e-4 absolute error of
// dQ/dK.  float32 tensors therefore carry the logits (and the subtraction of the
// running maximum / log-sum-exp) in float64, whose FMA issues at the same rate
// as unpacked float32 on this GPU; 16-bit tensors keep float32.
template <typename T> struct LogitAcc { using type = float; };
template <> struct LogitAcc<float> { using type = double; };

// exp(x) for x <= 0 through the hardware 2^y.  With float64 logits the float32
// rounding of y = x * log2(e) (up to 4e-6 for |y| ~ 60) is put back to first
// order: 2^(hi + lo) = 2^hi * (1 + lo * ln 2).
__device__ inline float exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ inline float exp_neg(double x) {
    const double y = fmax(x * 1.4426950408889634, -200.0);  // also maps -inf to an exact 0
    const float hi = (float)y;
    const float lo = (float)(y - (double)hi);
    const float e = __builtin_amdgcn_exp2f(hi);
    return fmaf(e, lo * 0.6931471805599453f, e);
}

constexpr int tile_w(int qpw) {
    int lg = 0;
    while ((1 << lg) < qpw) lg++;
    return 1 << ((lg + 1) / 2);
}

// Position of this lane group's pixel: workgroups tile each (batch, head) image
// with TH x TW blocks of pixels, or with runs of TH*TW positions when the image
// has a single row (the 1D operator).
template <int G>
struct Place {
    static constexpr int QPW = 256 / G;
    static constexpr int TW = tile_w(QPW);
    static constexpr int TH = QPW / TW;
    int b, n, x, y, lg;
    bool live;
    __device__ Place(const Shape &s, int tiles_y, int tiles_x) {
        int t = blockIdx.x;
        const int ty = t % tiles_y; t /= tiles_y;
        const int tx = t % tiles_x;
        const int slab = t / tiles_x;
        b = slab / s.N; n = slab % s.N;
        const int qi = threadIdx.x / G;
        lg = threadIdx.x % G;
        if (s.H == 1) {
            x = 0;
            y = ty * QPW + qi;
        } else {
            x = tx * TH + qi / TW;
            y = ty * TW + qi % TW;
        }
        live = x < s.H && y < s.W;
        x = min(x, s.H - 1);
        y = min(y, s.W - 1);
    }
};

template <typename T>
__device__ inline const T *at(const View &v, int b, int n, int x, int y) {
    return static_cast<const T *>(v.ptr) + b * v.sb + n * v.sn + x * v.sh + y * v.sw;
}

// Relative position bias of (query, key): entry (key - query + k - 1) per axis of the
// head's [2*kh-1, 2*kw-1] table (NATTEN's rule; the reference has no bias).
template <typename T>
__device__ inline float rpb_at(const void *rpb, const Shape &s, int n, int qx, int qy, int kx, int ky) {
    const int a = kx - qx + s.kh - 1, b = ky - qy + s.kw - 1;
    return cvt_in(static_cast<const T *>(rpb)[((int64_t)n * (2 * s.kh - 1) + a) * (2 * s.kw - 1) + b]);
}

// ---------------------------------------------------------------- forward
template <typename T, int G, int CH, bool VEC>
__global__ __launch_bounds__(256) void fwd_simt(FwdArgs a, int tiles_x, int tiles_y) {
    const Shape &s = a.s;
    const Place<G> pl(s, tiles_y, tiles_x);
    const int x0 = axis_start(pl.x, s.H, s.kh, s.ch), y0 = axis_start(pl.y, s.W, s.kw, s.cw);
    const int nx = axis_count(pl.x, s.H, s.kh, s.ch), ny = axis_count(pl.y, s.W, s.kw, s.cw);

    float qr[CH][8], acc[CH][8];
    const T *qp = at<T>(a.q, pl.b, pl.n, pl.x, pl.y);
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
        load8<T, VEC>(qp + d0, s.D - d0, qr[c]);
#pragma unroll
        for (int e = 0; e < 8; e++) acc[c][e] = 0.f;
    }
    using A = typename LogitAcc<T>::type;
    A m = -INFINITY;
    float l = 0.f;
    for (int i = 0; i < nx; i++) {
        for (int j = 0; j < ny; j++) {
            const T *kp = at<T>(a.k, pl.b, pl.n, x0 + i, y0 + j);
            const T *vp = at<T>(a.v, pl.b, pl.n, x0 + i, y0 + j);
            A part = 0;
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int d0 = (c * G + pl.lg) * 8;
                float kr[8];
                load8<T, VEC>(kp + d0, s.D - d0, kr);
#pragma unroll
                for (int e = 0; e < 8; e++) part = fma((A)qr[c][e], (A)kr[e], part);
            }
            A sc = group_sum<G>(part) * (A)s.scale;
            if (a.rpb) sc += (A)rpb_at<T>(a.rpb, s, pl.n, pl.x, pl.y, x0 + i, y0 + j);
            const A mn = sc > m ? sc : m;
            const float corr = exp_neg(m - mn);
            const float pj = exp_neg(sc - mn);
            l = l * corr + pj;
            m = mn;
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int d0 = (c * G + pl.lg) * 8;
                float vr[8];
                load8<T, VEC>(vp + d0, s.D - d0, vr);
#pragma unroll
                for (int e = 0; e < 8; e++) acc[c][e] = fmaf(pj, vr[e], acc[c][e] * corr);
            }
        }
    }
    if (!pl.live) return;
    const float inv = 1.f / l;
    const int64_t tok = (((int64_t)pl.b * s.N + pl.n) * s.H + pl.x) * s.W + pl.y;
    T *op = const_cast<T *>(at<T>(a.o, pl.b, pl.n, pl.x, pl.y));
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[c][e] *= inv;
        store8<T, VEC>(op + d0, s.D - d0, acc[c]);
    }
    if (a.lse && pl.lg == 0) a.lse[tok] = (float)(m + (A)logf(l));
}

// ---------------------------------------------------------------- dQ (+ delta)
template <typename T, int G, int CH, bool VEC>
__global__ __launch_bounds__(256) void bwd_dq_simt(BwdArgs a, int tiles_x, int tiles_y) {
    const Shape &s = a.s;
    const Place<G> pl(s, tiles_y, tiles_x);
    const int x0 = axis_start(pl.x, s.H, s.kh, s.ch), y0 = axis_start(pl.y, s.W, s.kw, s.cw);
    const int nx = axis_count(pl.x, s.H, s.kh, s.ch), ny = axis_count(pl.y, s.W, s.kw, s.cw);
    const int64_t tok = (((int64_t)pl.b * s.N + pl.n) * s.H + pl.x) * s.W + pl.y;

    float qr[CH][8], gr[CH][8], acc[CH][8], pk[CH][8];
    const T *qp = at<T>(a.q, pl.b, pl.n, pl.x, pl.y);
    const T *gp = at<T>(a.d_o, pl.b, pl.n, pl.x, pl.y);
    const T *op = at<T>(a.o, pl.b, pl.n, pl.x, pl.y);
    float dpart = 0.f;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
        float orow[8];
        load8<T, VEC>(qp + d0, s.D - d0, qr[c]);
        load8<T, VEC>(gp + d0, s.D - d0, gr[c]);
        load8<T, VEC>(op + d0, s.D - d0, orow);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            dpart = fmaf(gr[c][e], orow[e], dpart);
            acc[c][e] = 0.f;
            pk[c][e] = 0.f;
        }
    }
    // delta = dO . O centres dP; the probabilities recomputed from the stored
    // log-sum-exp carry a common factor (1 + eps) from its float32 rounding, so
    // their sum Z and the residual E = sum p (dP - delta) are accumulated too and
    // the result is renormalised exactly at the end:
    //   dQ = (A - (E / Z) * sum p k) / Z,  A = sum p (dP - delta) k.
    using A = typename LogitAcc<T>::type;
    const float delta = group_sum<G>(dpart);
    const A lse = a.lse[tok];
    float zsum = 0.f, esum = 0.f;
    for (int i = 0; i < nx; i++) {
        for (int j = 0; j < ny; j++) {
            const T *kp = at<T>(a.k, pl.b, pl.n, x0 + i, y0 + j);
            const T *vp = at<T>(a.v, pl.b, pl.n, x0 + i, y0 + j);
            float kr[CH][8];
            A ps = 0;
            float pd = 0.f;
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int d0 = (c * G + pl.lg) * 8;
                float vr[8];
                load8<T, VEC>(kp + d0, s.D - d0, kr[c]);
                load8<T, VEC>(vp + d0, s.D - d0, vr);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    ps = fma((A)qr[c][e], (A)kr[c][e], ps);
                    pd = fmaf(gr[c][e], vr[e], pd);
                }
            }
            A sl = group_sum<G>(ps) * (A)s.scale;
            if (a.rpb) sl += (A)rpb_at<T>(a.rpb, s, pl.n, pl.x, pl.y, x0 + i, y0 + j);
            const float p = exp_neg(sl - lse);
            const float ds = p * (group_sum<G>(pd) - delta);
            zsum += p;
            esum += ds;
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    acc[c][e] = fmaf(ds, kr[c][e], acc[c][e]);
                    pk[c][e] = fmaf(p, kr[c][e], pk[c][e]);
                }
        }
    }
    if (!pl.live) return;
    const float zinv = 1.f / zsum;
    const float shift = esum * zinv;
    T *dqp = static_cast<T *>(a.dq) + a.grad_at(pl.b, pl.n, pl.x, pl.y);  // (pl.x is the row)
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[c][e] = (acc[c][e] - shift * pk[c][e]) * (zinv * s.scale);
        store8<T, VEC>(dqp + d0, s.D - d0, acc[c]);
    }
    if (pl.lg == 0) {
        a.delta[tok] = delta + shift;
        a.zinv[tok] = zinv;
    }
}

// ---------------------------------------------------------------- dK, dV
// One lane group per key; it walks the queries that attend to the key
// (e_natten/pytorch.py:261-270) and needs delta and 1/Z from bwd_dq_simt.
template <typename T, int G, int CH, bool VEC>
__global__ __launch_bounds__(256) void bwd_dkdv_simt(BwdArgs a, int tiles_x, int tiles_y) {
    const Shape &s = a.s;
    const Place<G> pl(s, tiles_y, tiles_x);
    const int qx0 = axis_inv_lo(pl.x, s.kh, s.ch), qx1 = axis_inv_hi(pl.x, s.H, s.kh, s.ch);
    const int qy0 = axis_inv_lo(pl.y, s.kw, s.cw), qy1 = axis_inv_hi(pl.y, s.W, s.kw, s.cw);

    float kr[CH][8], vr[CH][8], dk[CH][8], dv[CH][8];
    const T *kp = at<T>(a.k, pl.b, pl.n, pl.x, pl.y);
    const T *vp = at<T>(a.v, pl.b, pl.n, pl.x, pl.y);
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
        load8<T, VEC>(kp + d0, s.D - d0, kr[c]);
        load8<T, VEC>(vp + d0, s.D - d0, vr[c]);
#pragma unroll
        for (int e = 0; e < 8; e++) { dk[c][e] = 0.f; dv[c][e] = 0.f; }
    }
    using A = typename LogitAcc<T>::type;
    const int64_t img = ((int64_t)pl.b * s.N + pl.n) * s.H * (int64_t)s.W;
    for (int xi = qx0; xi < qx1; xi++) {
        for (int yi = qy0; yi < qy1; yi++) {
            const int64_t qtok = img + (int64_t)xi * s.W + yi;
            const T *qp = at<T>(a.q, pl.b, pl.n, xi, yi);
            const T *gp = at<T>(a.d_o, pl.b, pl.n, xi, yi);
            float qr[CH][8], gr[CH][8];
            A ps = 0;
            float pd = 0.f;
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const int d0 = (c * G + pl.lg) * 8;
                load8<T, VEC>(qp + d0, s.D - d0, qr[c]);
                load8<T, VEC>(gp + d0, s.D - d0, gr[c]);
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    ps = fma((A)qr[c][e], (A)kr[c][e], ps);
                    pd = fmaf(gr[c][e], vr[c][e], pd);
                }
            }
            A sl = group_sum<G>(ps) * (A)s.scale;
            if (a.rpb) sl += (A)rpb_at<T>(a.rpb, s, pl.n, xi, yi, pl.x, pl.y);
            const float p = exp_neg(sl - (A)a.lse[qtok]) * a.zinv[qtok];
            const float ds = p * (group_sum<G>(pd) - a.delta[qtok]);
            // d(bias) of this (query, key) pair is dS itself; here P and dS are final (the
            // dQ pass left 1 / Z and the corrected delta).  It is left at the pair's place in
            // the query's window (every place is written exactly once, by the one key it
            // names), and rpb_grad_reduce sums the places of a bias entry in a fixed order.
            if (a.ds_pairs && pl.live && pl.lg == 0)
                a.ds_pairs[qtok * (s.kh * s.kw) + (pl.x - win_start(xi, s.H, s.kh)) * s.kw +
                           (pl.y - win_start(yi, s.W, s.kw))] = ds;
#pragma unroll
            for (int c = 0; c < CH; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    dk[c][e] = fmaf(ds, qr[c][e], dk[c][e]);
                    dv[c][e] = fmaf(p, gr[c][e], dv[c][e]);
                }
        }
    }
    if (!pl.live) return;
    const int64_t goff = a.grad_at(pl.b, pl.n, pl.x, pl.y);
    T *dkp = static_cast<T *>(a.dk) + goff;
    T *dvp = static_cast<T *>(a.dv) + goff;
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int d0 = (c * G + pl.lg) * 8;
#pragma unroll
        for (int e = 0; e < 8; e++) dk[c][e] *= s.scale;
        store8<T, VEC>(dkp + d0, s.D - d0, dk[c]);
        store8<T, VEC>(dvp + d0, s.D - d0, dv[c]);
    }
}

// Gradient of the relative position bias: entry (n, dy, dx) is the sum of dS over every
// (query, key) pair of head n with key - query = (dy, dx) (NATTEN's rule; the reference has
// no bias).  One workgroup per entry walks all queries of the head in a fixed order, each
// thread a strided share, and adds the 256 partial sums in a fixed tree: the same bits on
// every run, where adding the pairs with atomics as they are formed does not give that.
__global__ __launch_bounds__(256) void rpb_grad_reduce(const float *ds_pairs, float *d_rpb, Shape s) {
    __shared__ float part[256];
    const int EW = 2 * s.kw - 1, E = (2 * s.kh - 1) * EW;
    const int n = blockIdx.x / E, e = blockIdx.x % E;
    const int dy = e / EW - (s.kh - 1), dx = e % EW - (s.kw - 1);
    const int64_t hw = (int64_t)s.H * s.W, total = (int64_t)s.B * hw;
    float acc = 0.f;
    for (int64_t idx = threadIdx.x; idx < total; idx += 256) {
        const int b = (int)(idx / hw);
        const int pix = (int)(idx % hw), x = pix / s.W, y = pix % s.W;
        const int jx = x + dy - win_start(x, s.H, s.kh), jy = y + dx - win_start(y, s.W, s.kw);
        if ((unsigned)jx < (unsigned)s.kh && (unsigned)jy < (unsigned)s.kw)
            acc += ds_pairs[(((int64_t)b * s.N + n) * hw + pix) * (s.kh * s.kw) + jx * s.kw + jy];
    }
    part[threadIdx.x] = acc;
    __syncthreads();
    for (int w = 128; w > 0; w >>= 1) {
        if ((int)threadIdx.x < w) part[threadIdx.x] += part[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) d_rpb[blockIdx.x] = part[0];
}

// ---------------------------------------------------------------- dispatch
bool vec_ok(const View &v) {
    return (reinterpret_cast<uintptr_t>(v.ptr) % 16 == 0) && v.sb % 8 == 0 && v.sn % 8 == 0 &&
           v.sh % 8 == 0 && v.sw % 8 == 0;
}
bool vec_ok(const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return ENATTEN_ELAUNCH;
    }
    return ENATTEN_OK;
}

template <int G>
dim3 grid_for(const Shape &s, int &tiles_x, int &tiles_y) {
    if (s.H == 1) {
        tiles_x = 1;
        tiles_y = (s.W + Place<G>::QPW - 1) / Place<G>::QPW;
    } else {
        tiles_x = (s.H + Place<G>::TH - 1) / Place<G>::TH;
        tiles_y = (s.W + Place<G>::TW - 1) / Place<G>::TW;
    }
    return dim3((unsigned)((int64_t)s.B * s.N * tiles_x * tiles_y));
}

template <typename T, int G, int CH>
int fwd_cfg(const FwdArgs &a, bool vec, hipStream_t st) {
    int tx, ty;
    const dim3 grid = grid_for<G>(a.s, tx, ty);
    {
        ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_simt", st);
        if (vec) hipLaunchKernelGGL((fwd_simt<T, G, CH, true>), grid, dim3(256), 0, st, a, tx, ty);
        else hipLaunchKernelGGL((fwd_simt<T, G, CH, false>), grid, dim3(256), 0, st, a, tx, ty);
    }
    return check_launch("enatten2d_fwd");
}

template <typename T, int G, int CH>
int bwd_cfg(const BwdArgs &a, bool vec, hipStream_t st) {
    int tx, ty;
    const dim3 grid = grid_for<G>(a.s, tx, ty);
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_simt", st);
        if (vec) hipLaunchKernelGGL((bwd_dq_simt<T, G, CH, true>), grid, dim3(256), 0, st, a, tx, ty);
        else hipLaunchKernelGGL((bwd_dq_simt<T, G, CH, false>), grid, dim3(256), 0, st, a, tx, ty);
    }
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd_dkdv_simt", st);
        if (vec) hipLaunchKernelGGL((bwd_dkdv_simt<T, G, CH, true>), grid, dim3(256), 0, st, a, tx, ty);
        else hipLaunchKernelGGL((bwd_dkdv_simt<T, G, CH, false>), grid, dim3(256), 0, st, a, tx, ty);
    }
    if (a.d_rpb)
        hipLaunchKernelGGL(rpb_grad_reduce, dim3((unsigned)(a.s.N * (2 * a.s.kh - 1) * (2 * a.s.kw - 1))),
                           dim3(256), 0, st, a.ds_pairs, a.d_rpb, a.s);
    return check_launch("enatten2d_bwd");
}

// smallest lane group whose 8-channel slots cover D
#define ENATTEN_BY_D(FN, T, ARGS, VEC, ST)                        \
    do {                                                          \
        const int D_ = (ARGS).s.D;                                \
        if (D_ <= 8) return FN<T, 1, 1>(ARGS, VEC, ST);           \
        if (D_ <= 16) return FN<T, 2, 1>(ARGS, VEC, ST);          \
        if (D_ <= 32) return FN<T, 4, 1>(ARGS, VEC, ST);          \
        if (D_ <= 64) return FN<T, 8, 1>(ARGS, VEC, ST);          \
        if (D_ <= 128) return FN<T, 16, 1>(ARGS, VEC, ST);        \
        if (D_ <= 256) return FN<T, 32, 1>(ARGS, VEC, ST);        \
        if (D_ <= 512) return FN<T, 64, 1>(ARGS, VEC, ST);        \
        return FN<T, 64, 2>(ARGS, VEC, ST);                       \
    } while (0)

template <typename T>
int fwd_t(const FwdArgs &a, hipStream_t st) {
    const bool vec = a.s.D % 8 == 0 && vec_ok(a.q) && vec_ok(a.k) && vec_ok(a.v) && vec_ok(a.o);
    ENATTEN_BY_D(fwd_cfg, T, a, vec, st);
}
template <typename T>
int bwd_t(const BwdArgs &a, hipStream_t st) {
    const bool vec = a.s.D % 8 == 0 && vec_ok(a.q) && vec_ok(a.k) && vec_ok(a.v) && vec_ok(a.o) &&
                     vec_ok(a.d_o) && vec_ok(a.dq) && vec_ok(a.dk) && vec_ok(a.dv) && a.gsb % 8 == 0 &&
                     a.gsn % 8 == 0 && a.gsh % 8 == 0 && a.gsw % 8 == 0;
    ENATTEN_BY_D(bwd_cfg, T, a, vec, st);
}

}  // namespace

int launch_fwd_simt(const FwdArgs &a, int dtype, hipStream_t st) {
    if (a.s.D > 1024) {
        set_error("head dim %d exceeds the supported maximum of 1024", a.s.D);
        return ENATTEN_EUNSUPPORTED;
    }
    switch (dtype) {
        case ENATTEN_F32: return fwd_t<float>(a, st);
        case ENATTEN_BF16: return fwd_t<bf16_t>(a, st);
        case ENATTEN_F16: return fwd_t<f16_t>(a, st);
    }
    set_error("unknown dtype %d", dtype);
    return ENATTEN_EINVAL;
}

int launch_bwd_simt(const BwdArgs &a, int dtype, hipStream_t st) {
    if (a.s.D > 1024) {
        set_error("head dim %d exceeds the supported maximum of 1024", a.s.D);
        return ENATTEN_EUNSUPPORTED;
    }
    switch (dtype) {
        case ENATTEN_F32: return bwd_t<float>(a, st);
        case ENATTEN_BF16: return bwd_t<bf16_t>(a, st);
        case ENATTEN_F16: return bwd_t<f16_t>(a, st);
    }
    set_error("unknown dtype %d", dtype);
    return ENATTEN_EINVAL;
}

}  // namespace enatten
