// float64 neighborhood attention: plain double arithmetic end to end, for numerical
// gradient checks of the operator itself (the reference's only gradient check runs in
// double, gradcheck.py:6-15) and for callers that hold float64 tensors.  Not tuned: one
// wave per query (or key), each lane a strided share of the channels, dot products
// finished with shuffles, K / V (Q / dO) rows straight from global memory.
//
// Per-query math: e_natten/pytorch.py:196-202 (forward), :248-288 (backward), with the
// softmax Jacobian product written as dS = P * (dP - dO . O).  The backward recomputes every
// query's own log-sum-exp in double (the float32 one that the forward hands out would put
// 1e-7 on every probability) and leaves it, with dO . O, in the workspace for the dK/dV pass:
// two doubles per query.  Windows: any extent per axis, centred or causal, as in the general
// kernels; no relative position bias.

#include <math.h>

#include "na2d_common.h"

namespace enatten {
namespace {

__device__ inline double wave_sum(double x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

struct Pixel {
    int b, n, y, x;
    int64_t tok;
    bool live;
};
__device__ inline Pixel pixel_of_wave(const Shape &s) {
    Pixel p;
    const int64_t t = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t total = (int64_t)s.B * s.N * s.H * s.W;
    p.live = t < total;
    p.tok = p.live ? t : total - 1;
    int64_t r = p.tok;
    p.x = (int)(r % s.W); r /= s.W;
    p.y = (int)(r % s.H); r /= s.H;
    p.n = (int)(r % s.N);
    p.b = (int)(r / s.N);
    return p;
}
__device__ inline const double *row_of(const View &v, int b, int n, int y, int x) {
    return static_cast<const double *>(v.ptr) + b * v.sb + n * v.sn + y * v.sh + x * v.sw;
}

// NCH: channels per lane, D <= 64 * NCH
template <int NCH>
__device__ inline void load_row(const double *p, int D, int lane, double (&r)[NCH]) {
#pragma unroll
    for (int i = 0; i < NCH; i++) r[i] = lane + 64 * i < D ? p[lane + 64 * i] : 0.0;
}
template <int NCH>
__device__ inline double dot_row(const double *p, int D, int lane, const double (&a)[NCH]) {
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if (lane + 64 * i < D) acc = fma(a[i], p[lane + 64 * i], acc);
    return wave_sum(acc);
}

template <int NCH>
__global__ __launch_bounds__(256) void fwd_f64(FwdArgs a) {
    const Shape &s = a.s;
    const Pixel px = pixel_of_wave(s);
    const int lane = threadIdx.x & 63;
    double q[NCH], acc[NCH];
    load_row<NCH>(row_of(a.q, px.b, px.n, px.y, px.x), s.D, lane, q);
#pragma unroll
    for (int i = 0; i < NCH; i++) acc[i] = 0.0;
    const int ys = axis_start(px.y, s.H, s.kh, s.ch), yn = axis_count(px.y, s.H, s.kh, s.ch);
    const int xs = axis_start(px.x, s.W, s.kw, s.cw), xn = axis_count(px.x, s.W, s.kw, s.cw);
    double m = -INFINITY, l = 0.0;
    for (int r = ys; r < ys + yn; r++)
        for (int c = xs; c < xs + xn; c++) {
            const double sj = dot_row<NCH>(row_of(a.k, px.b, px.n, r, c), s.D, lane, q) * (double)s.scale;
            const double mn = fmax(m, sj), corr = exp(m - mn), p = exp(sj - mn);
            const double *vp = row_of(a.v, px.b, px.n, r, c);
            l = l * corr + p;
#pragma unroll
            for (int i = 0; i < NCH; i++)
                if (lane + 64 * i < s.D) acc[i] = acc[i] * corr + p * vp[lane + 64 * i];
            m = mn;
        }
    if (!px.live) return;
    double *op = const_cast<double *>(row_of(a.o, px.b, px.n, px.y, px.x));
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if (lane + 64 * i < s.D) op[lane + 64 * i] = acc[i] / l;
    if (a.lse && lane == 0) a.lse[px.tok] = (float)(m + log(l));
}

// dQ, and (log-sum-exp, dO . O) of the query in double for the dK/dV pass
template <int NCH>
__global__ __launch_bounds__(256) void bwd_dq_f64(BwdArgs a, double2 *stat) {
    const Shape &s = a.s;
    const Pixel px = pixel_of_wave(s);
    const int lane = threadIdx.x & 63;
    double q[NCH], g[NCH], dq[NCH];
    load_row<NCH>(row_of(a.q, px.b, px.n, px.y, px.x), s.D, lane, q);
    load_row<NCH>(row_of(a.d_o, px.b, px.n, px.y, px.x), s.D, lane, g);
    const double delta = dot_row<NCH>(row_of(a.o, px.b, px.n, px.y, px.x), s.D, lane, g);
#pragma unroll
    for (int i = 0; i < NCH; i++) dq[i] = 0.0;
    const int ys = axis_start(px.y, s.H, s.kh, s.ch), yn = axis_count(px.y, s.H, s.kh, s.ch);
    const int xs = axis_start(px.x, s.W, s.kw, s.cw), xn = axis_count(px.x, s.W, s.kw, s.cw);
    double m = -INFINITY, l = 0.0;
    for (int r = ys; r < ys + yn; r++)
        for (int c = xs; c < xs + xn; c++) {
            const double sj = dot_row<NCH>(row_of(a.k, px.b, px.n, r, c), s.D, lane, q) * (double)s.scale;
            const double mn = fmax(m, sj);
            l = l * exp(m - mn) + exp(sj - mn);
            m = mn;
        }
    const double lse = m + log(l);
    for (int r = ys; r < ys + yn; r++)
        for (int c = xs; c < xs + xn; c++) {
            const double *kp = row_of(a.k, px.b, px.n, r, c);
            const double sj = dot_row<NCH>(kp, s.D, lane, q) * (double)s.scale;
            const double p = exp(sj - lse);
            const double dp = dot_row<NCH>(row_of(a.v, px.b, px.n, r, c), s.D, lane, g);
            const double ds = p * (dp - delta);
#pragma unroll
            for (int i = 0; i < NCH; i++)
                if (lane + 64 * i < s.D) dq[i] = fma(ds, kp[lane + 64 * i], dq[i]);
        }
    if (!px.live) return;
    double *out = static_cast<double *>(a.dq) + a.grad_at(px.b, px.n, px.y, px.x);
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if (lane + 64 * i < s.D) out[lane + 64 * i] = dq[i] * (double)s.scale;
    if (lane == 0) stat[px.tok] = make_double2(lse, delta);
}

// dK, dV of one key over the queries whose window holds it: per axis exactly
// [axis_inv_lo, axis_inv_hi) (e_natten/pytorch.py:13-23), no atomics
template <int NCH>
__global__ __launch_bounds__(256) void bwd_dkdv_f64(BwdArgs a, const double2 *stat) {
    const Shape &s = a.s;
    const Pixel px = pixel_of_wave(s);
    const int lane = threadIdx.x & 63;
    double k[NCH], v[NCH], dk[NCH], dv[NCH];
    load_row<NCH>(row_of(a.k, px.b, px.n, px.y, px.x), s.D, lane, k);
    load_row<NCH>(row_of(a.v, px.b, px.n, px.y, px.x), s.D, lane, v);
#pragma unroll
    for (int i = 0; i < NCH; i++) dk[i] = dv[i] = 0.0;
    const int y0 = axis_inv_lo(px.y, s.kh, s.ch), y1 = axis_inv_hi(px.y, s.H, s.kh, s.ch);
    const int x0 = axis_inv_lo(px.x, s.kw, s.cw), x1 = axis_inv_hi(px.x, s.W, s.kw, s.cw);
    const int64_t img = ((int64_t)px.b * s.N + px.n) * s.H * (int64_t)s.W;
    for (int r = y0; r < y1; r++)
        for (int c = x0; c < x1; c++) {
            const double *qp = row_of(a.q, px.b, px.n, r, c), *gp = row_of(a.d_o, px.b, px.n, r, c);
            const double2 st = stat[img + (int64_t)r * s.W + c];
            const double sj = dot_row<NCH>(qp, s.D, lane, k) * (double)s.scale;
            const double p = exp(sj - st.x);
            const double dp = dot_row<NCH>(gp, s.D, lane, v);
            const double ds = p * (dp - st.y);
#pragma unroll
            for (int i = 0; i < NCH; i++)
                if (lane + 64 * i < s.D) {
                    dv[i] = fma(p, gp[lane + 64 * i], dv[i]);
                    dk[i] = fma(ds, qp[lane + 64 * i], dk[i]);
                }
        }
    if (!px.live) return;
    const int64_t goff = a.grad_at(px.b, px.n, px.y, px.x);
    double *okp = static_cast<double *>(a.dk) + goff, *ovp = static_cast<double *>(a.dv) + goff;
#pragma unroll
    for (int i = 0; i < NCH; i++)
        if (lane + 64 * i < s.D) {
            okp[lane + 64 * i] = dk[i] * (double)s.scale;
            ovp[lane + 64 * i] = dv[i];
        }
}

int check(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return ENATTEN_ELAUNCH;
    }
    return ENATTEN_OK;
}

// grid: one wave per pixel, four to a workgroup
bool grid_of(const Shape &s, unsigned *grid) {
    const int64_t blocks = ((int64_t)s.B * s.N * s.H * s.W + 3) / 4;
    if (blocks > 0x7fffffff) {
        set_error("float64 kernels: more than 2^33 pixels");
        return false;
    }
    *grid = (unsigned)blocks;
    return true;
}

#define ENATTEN_F64_BY_D(KERNEL, ...)                                                        \
    do {                                                                                     \
        const int nch = (a.s.D + 63) / 64;                                                   \
        if (nch <= 1) hipLaunchKernelGGL((KERNEL<1>), dim3(grid), dim3(256), 0, st, __VA_ARGS__);       \
        else if (nch <= 2) hipLaunchKernelGGL((KERNEL<2>), dim3(grid), dim3(256), 0, st, __VA_ARGS__);  \
        else if (nch <= 4) hipLaunchKernelGGL((KERNEL<4>), dim3(grid), dim3(256), 0, st, __VA_ARGS__);  \
        else if (nch <= 8) hipLaunchKernelGGL((KERNEL<8>), dim3(grid), dim3(256), 0, st, __VA_ARGS__);  \
        else hipLaunchKernelGGL((KERNEL<16>), dim3(grid), dim3(256), 0, st, __VA_ARGS__);               \
    } while (0)

}  // namespace

int launch_fwd_f64(const FwdArgs &a, hipStream_t st) {
    if (a.rpb) {
        set_error("float64 tensors: no relative position bias");
        return ENATTEN_EUNSUPPORTED;
    }
    unsigned grid;
    if (!grid_of(a.s, &grid)) return ENATTEN_EUNSUPPORTED;
    {
        ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_f64", st);
        ENATTEN_F64_BY_D(fwd_f64, a);
    }
    return check("float64 forward");
}

// a.delta: 2 doubles (4 floats) per query, 16-byte aligned
int launch_bwd_f64(const BwdArgs &a, hipStream_t st) {
    if (a.rpb) {
        set_error("float64 tensors: no relative position bias");
        return ENATTEN_EUNSUPPORTED;
    }
    if (reinterpret_cast<uintptr_t>(a.delta) % 16 != 0) {
        set_error("float64 backward: the workspace must be 16-byte aligned");
        return ENATTEN_EINVAL;
    }
    unsigned grid;
    if (!grid_of(a.s, &grid)) return ENATTEN_EUNSUPPORTED;
    double2 *stat = reinterpret_cast<double2 *>(a.delta);
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_f64", st);
        ENATTEN_F64_BY_D(bwd_dq_f64, a, stat);
    }
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd_dkdv_f64", st);
        ENATTEN_F64_BY_D(bwd_dkdv_f64, a, stat);
    }
    return check("float64 backward");
}

}  // namespace enatten
