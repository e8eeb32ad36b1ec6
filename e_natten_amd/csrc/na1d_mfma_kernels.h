// Matrix-core (MFMA) kernels for 1D neighborhood attention on gfx950.
//
// A sequence is cut into tiles of 64 consecutive positions; a workgroup of four waves
// owns a tile, each wave 16 positions (the N dimension of v_mfma_f32_16x16x32).  The
// keys that the wave's 16 queries can see are the 16 + k - 1 consecutive positions from
// the window start of its first query on; they are the MFMA rows of the first product
// (S^T = K Q^T), padded to NKP = 32 tokens for kernel_size <= 17 and 64 for
// kernel_size <= 49.  The rows of K and V that the tile needs (64 + k - 1 positions)
// are staged in LDS once per tile with coalesced 16-byte loads; the next tile's rows
// are in flight into registers while the current one is computed.  Everything else is
// the scheme of the 2D kernels (na2d_mfma_kernels.h): every lane holds the logits of one
// query for several keys, the reduction index of the second product is enumerated in
// the order the accumulators hold it, and its other operand comes out of LDS through
// the transposing read.  The kernel size is a run-time argument: a token's place in
// LDS is (first row of the wave) + (token number), and the mask is one comparison.
//
// The dK/dV pass is key-centric: a wave owns 16 keys and walks the queries that attend
// to any of them (e_natten/pytorch.py:13-23, :124-152), 32 at a time; no atomics.
//
// Per-query math: e_natten/triton.py:65-222 (1D kernels), :425-485 (host).
//
// Compiled twice, like the 2D kernels: na1d_mfma.hip (head dims 32, 64, 128 themselves) and
// na1d_mfma_narrow.hip (the other multiples of 8 up to 128) each define
// `enatten::(anonymous)::kNarrow` before including this file.

#include "na2d_mfma.h"

namespace enatten {
namespace {

template <int D, int NKP>
struct Geo1 {
    static constexpr int TW = 64;                  // positions per workgroup
    static constexpr int KSMAX = NKP - 15;         // largest kernel_size served
    static constexpr int HR = TW + KSMAX - 1;      // staged key rows (forward, dQ)
    static constexpr int RQ = TW + KSMAX - 1 + KSMAX / 2;  // staged query rows (dK/dV)
    static constexpr int PITCH = D + 8;            // LDS row pitch in elements (16-byte pad)
    static constexpr int MT = NKP / 16;            // 16-token MFMA row tiles
    static constexpr int KSTEPS = NKP / 32;        // reduction steps of the second product
    static constexpr int DS = D / 32;              // reduction steps over channels
    static constexpr int DT = D / 16;              // 16-channel row tiles of the output
};

// A tile of 64 positions of one (batch, head) sequence.
struct Tile1 {
    int bb, nn, t0;
};
__device__ __forceinline__ Tile1 tile1_of(int t, int tiles_t, int N) {
    Tile1 tl;
    tl.t0 = (t % tiles_t) * 64; t /= tiles_t;
    tl.nn = t % N; tl.bb = t / N;
    return tl;
}
__device__ __forceinline__ const short *seq(const View &v, const Tile1 &tl) {
    return static_cast<const short *>(v.ptr) + tl.bb * v.sb + tl.nn * v.sn;
}

// NR rows of a sequence from position p0 on (clamped to the last position: such rows
// only ever meet zero probabilities) into registers, then into LDS rows 0 .. NR-1.
template <int D, int NR>
struct Stage1 {
    static constexpr int CPR = D / 8, RPP = 256 / CPR, NL = (NR * CPR + 255) / 256;
    u32x4 v[NL];
    // dlim: the tensor's head dim (D, or less in the build for narrow head dims): a thread whose
    // channel chunk the tensor does not have moves nothing, and its LDS columns stay zero
    __device__ __forceinline__ void fetch(const short *sq, int64_t sw, int p0, int T, int dlim) {
        if (((int)threadIdx.x % CPR) * 8 >= dlim) {
            // (zero, not stale: the one-pass backward sums dO . O over the staged registers)
#pragma unroll
            for (int i = 0; i < NL; i++) v[i] = u32x4{0u, 0u, 0u, 0u};
            return;
        }
        const int pb = min(p0, T - 1);
        const char *base = reinterpret_cast<const char *>(sq + pb * sw);
        const unsigned sw2 = (unsigned)sw * 2u;
        const int rmax = T - 1 - pb;
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int r = min(min((int)threadIdx.x / CPR + i * RPP, NR - 1), rmax);
            const unsigned off = __umul24((unsigned)r, sw2) + ((unsigned)threadIdx.x % CPR) * 16u;
            v[i] = *reinterpret_cast<const u32x4 *>(base + off);
        }
    }
    __device__ __forceinline__ void commit(short *lds, int dlim) const {
        if (((int)threadIdx.x % CPR) * 8 >= dlim) return;
#pragma unroll
        for (int i = 0; i < NL; i++) {
            const int r = (int)threadIdx.x / CPR + i * RPP;
            if (r < NR)
                *reinterpret_cast<u32x4 *>(lds + r * (D + 8) + ((int)threadIdx.x % CPR) * 8) = v[i];
        }
    }
};

// The all-zero row `zrow` and, for a head dim below D, the channels from `dlim` on of the rows
// before it (no commit ever writes those).
template <int D>
__device__ __forceinline__ void zero_row1(short *lds, int zrow, int dlim) {
    if (threadIdx.x < D / 8)
        *reinterpret_cast<uint4 *>(lds + zrow * (D + 8) + threadIdx.x * 8) = make_uint4(0, 0, 0, 0);
    if (dlim < D) {
        const int c0 = dlim >> 3, npad = D / 8 - c0;
        for (int idx = threadIdx.x; idx < zrow * npad; idx += 256)
            *reinterpret_cast<uint4 *>(lds + (idx / npad) * (D + 8) + (c0 + idx % npad) * 8) = make_uint4(0, 0, 0, 0);
    }
}

// What a lane knows about its query (forward, dQ).
struct Lane1 {
    bool wave_on, live;
    int qt;     // query position, clamped into the sequence
    int orow;   // LDS row of the wave's first token
    int d;      // window start of this query relative to the wave's first token
    int hr0;    // first staged position
    int64_t tok;
};
__device__ __forceinline__ Lane1 lane1(const Tile1 &tl, const Shape &s, int wave, int n) {
    const int T = s.W, ks = s.kw;
    Lane1 q;
    const int w0 = tl.t0 + wave * 16;
    q.wave_on = w0 < T;
    q.live = w0 + n < T;
    q.qt = min(w0 + n, T - 1);
    q.hr0 = win_start(tl.t0, T, ks);
    const int sr0 = win_start(min(w0, T - 1), T, ks);
    q.orow = sr0 - q.hr0;
    q.d = win_start(q.qt, T, ks) - sr0;
    q.tok = ((int64_t)tl.bb * s.N + tl.nn) * T + q.qt;
    return q;
}

// ------------------------------------------------------------------ forward
template <bool BF, int D, int NKP>
__global__ __launch_bounds__(256, 2) void fwd1d_mfma(FwdArgs a, int tiles_t, int ntiles) {
    using G = Geo1<D, NKP>;
    __shared__ __attribute__((aligned(16))) short lds_k[(G::HR + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[(G::HR + 1) * G::PITCH];
    const Shape &s = a.s;
    const int T = s.W, ks = s.kw;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row1<D>(lds_k, G::HR, dlim);
    zero_row1<D>(lds_v, G::HR, dlim);
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const int ntok = 15 + ks;  // tokens of a wave

    Stage1<D, G::HR> kst, vst;
    s16x8 qnext[G::DS];
    auto prefetch = [&](const Tile1 &tl, const Lane1 &lq) __attribute__((always_inline)) {
        kst.fetch(seq(a.k, tl), a.k.sw, lq.hr0, T, dlim);
        vst.fetch(seq(a.v, tl), a.v.sw, lq.hr0, T, dlim);
        load_row_chunks(qnext, seq(a.q, tl) + lq.qt * a.q.sw, g, dlim);
    };
    Tile1 cur = tile1_of(sc.t, tiles_t, s.N);
    Lane1 lq = lane1(cur, s, wave, n);
    prefetch(cur, lq);
    for (;;) {
        kst.commit(lds_k, dlim);
        vst.commit(lds_v, dlim);
        s16x8 qreg[G::DS];
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) qreg[ds] = qnext[ds];
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        Tile1 nxt = cur;
        Lane1 lqn = lq;
        if (more) {
            nxt = tile1_of(tn, tiles_t, s.N);
            lqn = lane1(nxt, s, wave, n);
            prefetch(nxt, lqn);
        }
        auto trow = [&](int tk) __attribute__((always_inline)) {
            return tk < ntok ? lq.orow + tk : (int)G::HR;
        };
        if (lq.wave_on) {
            f32x4 acc[G::MT];
            float mx = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const short *kp = lds_k + trow(mt * 16 + n) * G::PITCH + g * 8;
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++)
                    c = mfma16<BF>(*reinterpret_cast<const s16x8 *>(kp + ds * 32), qreg[ds], c);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int tk = mt * 16 + g * 4 + i;
                    const bool ok = (unsigned)(tk - lq.d) < (unsigned)ks;
                    c[i] = ok ? c[i] * sc2 : -INFINITY;
                    mx = fmaxf(mx, c[i]);
                }
                acc[mt] = c;
            }
            mx = col_max(mx);
            float sum = 0.f;
            s16x8 pb[G::KSTEPS];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float p = __builtin_amdgcn_exp2f(acc[mt][i] - mx);
                    sum += p;
                    pb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                }
            sum = col_sum(sum);
            f32x4 o[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) o[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < G::KSTEPS; kk++) {
                const short *vp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    vp[h] = lds_v + trow(kk * 32 + h * 16 + g * 4 + (n >> 2)) * G::PITCH + (n & 3) * (D / 4);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    o[mt] = mfma16<BF>(cat(lds_read_tr(vp[0] + mt * 4), lds_read_tr(vp[1] + mt * 4)),
                                       pb[kk], o[mt]);
            }
            store_token<BF, D, D >= 64 && !kNarrow>(const_cast<short *>(seq(a.o, cur)) + lq.qt * a.o.sw, g, o, 1.f / sum,
                               lq.live, dlim);
            if (lq.live && a.lse && g == 0) a.lse[lq.tok] = (mx + __builtin_amdgcn_logf(sum)) * kLn2;
        }
        if (!more) break;
        __syncthreads();
        cur = nxt;
        lq = lqn;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dQ
// P from the saved log-sum-exp, dP^T = V dO^T, delta = sum_j P_j dP_j,
// dS = P (dP - delta), dQ^T = K^T dS^T; writes dQ and delta.
template <bool BF, int D, int NKP>
__global__ __launch_bounds__(256, 2) void bwd1d_dq_mfma(BwdArgs a, int tiles_t, int ntiles) {
    using G = Geo1<D, NKP>;
    __shared__ __attribute__((aligned(16))) short lds_k[(G::HR + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[(G::HR + 1) * G::PITCH];
    const Shape &s = a.s;
    const int T = s.W, ks = s.kw;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row1<D>(lds_k, G::HR, dlim);
    zero_row1<D>(lds_v, G::HR, dlim);
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const int ntok = 15 + ks;

    Stage1<D, G::HR> kst, vst;
    s16x8 qnext[G::DS], gnext[G::DS];
    float lse_next = 0.f;
    auto prefetch = [&](const Tile1 &tl, const Lane1 &lq) __attribute__((always_inline)) {
        kst.fetch(seq(a.k, tl), a.k.sw, lq.hr0, T, dlim);
        vst.fetch(seq(a.v, tl), a.v.sw, lq.hr0, T, dlim);
        load_row_chunks(qnext, seq(a.q, tl) + lq.qt * a.q.sw, g, dlim);
        load_row_chunks(gnext, seq(a.d_o, tl) + lq.qt * a.d_o.sw, g, dlim);
        lse_next = a.lse[lq.tok];
    };
    Tile1 cur = tile1_of(sc.t, tiles_t, s.N);
    Lane1 lq = lane1(cur, s, wave, n);
    prefetch(cur, lq);
    for (;;) {
        kst.commit(lds_k, dlim);
        vst.commit(lds_v, dlim);
        s16x8 qreg[G::DS], greg[G::DS];
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) {
            qreg[ds] = qnext[ds];
            greg[ds] = gnext[ds];
        }
        const float lse2 = lse_next * kLog2e;
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        Tile1 nxt = cur;
        Lane1 lqn = lq;
        if (more) {
            nxt = tile1_of(tn, tiles_t, s.N);
            lqn = lane1(nxt, s, wave, n);
            prefetch(nxt, lqn);
        }
        auto trow = [&](int tk) __attribute__((always_inline)) {
            return tk < ntok ? lq.orow + tk : (int)G::HR;
        };
        if (lq.wave_on) {
            f32x4 dp[G::MT];
            s16x8 dsb[G::KSTEPS];
            float dpart = 0.f;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const int row = trow(mt * 16 + n);
                const short *kp = lds_k + row * G::PITCH + g * 8, *vp = lds_v + row * G::PITCH + g * 8;
                f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(kp + ds * 32), qreg[ds], cs);
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(vp + ds * 32), greg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int tk = mt * 16 + g * 4 + i;
                    const bool ok = (unsigned)(tk - lq.d) < (unsigned)ks;
                    cs[i] = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - lse2 : -INFINITY);
                    dpart = fmaf(cs[i], cp[i], dpart);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(cs[i]);
                }
                dp[mt] = cp;
            }
            const float delta = col_sum(dpart);
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float p = cvt32<BF>(dsb[mt >> 1][(mt & 1) * 4 + i]);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (dp[mt][i] - delta));
                }
            f32x4 dq[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < G::KSTEPS; kk++) {
                const short *kp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    kp[h] = lds_k + trow(kk * 32 + h * 16 + g * 4 + (n >> 2)) * G::PITCH + (n & 3) * (D / 4);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    dq[mt] = mfma16<BF>(cat(lds_read_tr(kp[0] + mt * 4), lds_read_tr(kp[1] + mt * 4)),
                                        dsb[kk], dq[mt]);
            }
            store_token<BF, D, D >= 64 && !kNarrow>(static_cast<short *>(a.dq) + a.grad_at(cur.bb, cur.nn, 0, lq.qt), g, dq, s.scale, lq.live, dlim);
            if (lq.live && g == 0) a.delta[lq.tok] = delta;
        }
        if (!more) break;
        __syncthreads();
        cur = nxt;
        lq = lqn;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dK, dV
// The workgroup owns 64 keys and stages Q, dO, the log-sum-exp and delta of the queries
// that attend to any of them: [inv_lo(first key), inv_hi(last key)), at most
// 64 + k - 1 + k/2 positions (the clamped windows of the k/2 queries beside an end of the
// sequence all reach k positions in).  A wave owns 16 keys (MFMA columns) and walks the
// queries that can attend to them, 32 at a time:
//   S = Q K^T, dP = dO V^T, P = exp(S - lse), dS = P (dP - delta), masked to the
//   query's own window; dV^T += dO^T P, dK^T += Q^T dS.
template <bool BF, int D, int NKP>
__global__ __launch_bounds__(256, 2) void bwd1d_dkdv_mfma(BwdArgs a, int tiles_t, int ntiles) {
    using G = Geo1<D, NKP>;
    __shared__ __attribute__((aligned(16))) short lds_q[(G::RQ + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[(G::RQ + 1) * G::PITCH];
    __shared__ float2 lds_stat[G::RQ + 1];  // (lse * log2e, delta) per staged query
    const Shape &s = a.s;
    const int T = s.W, ks = s.kw;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row1<D>(lds_q, G::RQ, dlim);
    zero_row1<D>(lds_g, G::RQ, dlim);
    if (threadIdx.x == 0) lds_stat[G::RQ] = make_float2(0.f, 0.f);
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;

    Stage1<D, G::RQ> qst, gst;
    float2 sst = make_float2(0.f, 0.f);
    static_assert(G::RQ <= 256, "one statistics pair per thread");
    auto prefetch = [&](const Tile1 &tl) __attribute__((always_inline)) {
        const int qa = inv_lo(tl.t0, ks);
        qst.fetch(seq(a.q, tl), a.q.sw, qa, T, dlim);
        gst.fetch(seq(a.d_o, tl), a.d_o.sw, qa, T, dlim);
        const int64_t sq0 = ((int64_t)tl.bb * s.N + tl.nn) * T;
        const int qp = min(qa + min((int)threadIdx.x, G::RQ - 1), T - 1);
        sst = make_float2(a.lse[sq0 + qp] * kLog2e, a.delta[sq0 + qp]);
    };
    // B operands of a tile: this lane's key, channels ds*32 + g*8 ..  Loaded when the
    // previous tile's math is over (a second set would not fit beside it).
    s16x8 kreg[G::DS], vreg[G::DS];
    auto load_keys = [&](const Tile1 &tl) __attribute__((always_inline)) {
        const int kt = min(tl.t0 + wave * 16 + n, T - 1);
        load_row_chunks(kreg, seq(a.k, tl) + kt * a.k.sw, g, dlim);
        load_row_chunks(vreg, seq(a.v, tl) + kt * a.v.sw, g, dlim);
    };
    Tile1 cur = tile1_of(sc.t, tiles_t, s.N);
    prefetch(cur);
    load_keys(cur);
    for (;;) {
        qst.commit(lds_q, dlim);
        gst.commit(lds_g, dlim);
        if (threadIdx.x < G::RQ) lds_stat[threadIdx.x] = sst;
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        Tile1 nxt = cur;
        if (more) {
            nxt = tile1_of(tn, tiles_t, s.N);
            prefetch(nxt);
        }
        const int w0 = cur.t0 + wave * 16;
        const bool wave_on = w0 < T;
        const int kt = min(w0 + n, T - 1);
        f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
        for (int mt = 0; mt < G::DT; mt++) {
            dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        if (wave_on) {
            const int qa = inv_lo(cur.t0, ks);
            // this wave's queries: those that attend to any of its 16 keys
            const int wa = inv_lo(w0, ks), wb = inv_hi(min(w0 + 16, T) - 1, T, ks);
            const int nq = wb - wa, r0 = wa - qa;
            auto row_of = [&](int qi) __attribute__((always_inline)) {
                return qi < nq ? r0 + qi : (int)G::RQ;
            };
            for (int q0 = 0; q0 < nq; q0 += 32) {
                s16x8 pb, dsb;
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++) {
                    const int row = row_of(q0 + m2 * 16 + n);
                    const short *qp = lds_q + row * G::PITCH + g * 8, *gp = lds_g + row * G::PITCH + g * 8;
                    f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ds = 0; ds < G::DS; ds++) {
                        cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(qp + ds * 32), kreg[ds], cs);
                        cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(gp + ds * 32), vreg[ds], cp);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int qi = q0 + m2 * 16 + g * 4 + i;
                        const float2 st = lds_stat[row_of(qi)];
                        const bool ok = (qi < nq) &
                                        ((unsigned)(kt - win_start(wa + qi, T, ks)) < (unsigned)ks);
                        const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
                        pb[m2 * 4 + i] = cvt16<BF>(p);
                        dsb[m2 * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                    }
                }
                const short *qt[2], *gt[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int row = row_of(q0 + h * 16 + g * 4 + (n >> 2));
                    qt[h] = lds_q + row * G::PITCH + (n & 3) * (D / 4);
                    gt[h] = lds_g + row * G::PITCH + (n & 3) * (D / 4);
                }
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dv[mt] = mfma16<BF>(cat(lds_read_tr(gt[0] + mt * 4), lds_read_tr(gt[1] + mt * 4)), pb, dv[mt]);
                    dk[mt] = mfma16<BF>(cat(lds_read_tr(qt[0] + mt * 4), lds_read_tr(qt[1] + mt * 4)), dsb, dk[mt]);
                }
            }
            const int64_t goff = a.grad_at(cur.bb, cur.nn, 0, kt);
            const bool live = w0 + n < T;
            store_token<BF, D, D >= 64 && !kNarrow>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, live, dlim);
            store_token<BF, D, D >= 64 && !kNarrow>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, live, dlim);
        }
        if (!more) break;
        load_keys(nxt);
        __syncthreads();
        cur = nxt;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dQ, dK, dV in one pass
// The rows of q, k, v and dO that a tile of 64 positions needs, as queries' keys and as
// keys' queries, are staged ONCE: positions [row0, row0 + RQ), where row0 is the smaller of
// the window start of the tile's first query and the first query that attends its first
// key.  delta = dO . O of every staged query is formed while the rows are written to LDS
// (the forward output is read for this and for nothing else), so the backward reads five
// tensors and writes three where the two passes read eight and write three.  Each wave
// first forms dQ of its 16 positions (as bwd1d_dq_mfma), then dK and dV of the same 16
// positions (as bwd1d_dkdv_mfma), all operands out of LDS.
// Workgroups per CU that the registers are budgeted for: what LDS admits, at most three.
// (At head_dim 128 LDS holds one workgroup; a variant with eight waves there, four for dQ
// and four for dK and dV, was measured level with this one.)
// FULL: the sequence length is a multiple of the 64 positions of a tile, so every lane's
// position exists: no wave is switched off, no store is predicated, and the staged rows go to
// LDS at the end of a tile's pass through the loop instead of at the top of the next.  The
// compiler then knows how many stores lie between the loads of those rows and their use, and
// the wait for the rows does not wait for the tile's stores as well (see fwd_mfma of the 2D
// kernels).  Used at head_dim 128, where one workgroup per CU has nothing to cover that wait
// with (B8 N8 T8192 k13: 229.6 -> 221 us; at head_dim 64 it measured 91.9 -> 92.2).
template <bool BF, int D, int NKP, bool FULL = false>
__global__ __launch_bounds__(256, D == 32 ? 3 : D == 64 ? 2 : 1) void bwd1d_fused_mfma(
    BwdArgs a, int tiles_t, int ntiles) {
    using G = Geo1<D, NKP>;
    constexpr int NR = G::RQ, CPR = D / 8;
    __shared__ __attribute__((aligned(16))) short lds_q[(NR + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[(NR + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_k[(NR + 1) * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[(NR + 1) * G::PITCH];
    __shared__ float2 lds_stat[NR + 1];  // (lse * log2e, dO . O) per staged position
    const Shape &s = a.s;
    const int T = s.W, ks = s.kw;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row1<D>(lds_q, NR, dlim);
    zero_row1<D>(lds_g, NR, dlim);
    zero_row1<D>(lds_k, NR, dlim);
    zero_row1<D>(lds_v, NR, dlim);
    if (threadIdx.x == 0) lds_stat[NR] = make_float2(0.f, 0.f);
    const int wave = FULL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const int ntok = 15 + ks;

    using St = Stage1<D, NR>;
    St qst, gst, kst, vst, ost;
    float lse_st = 0.f;
    static_assert(NR <= 256, "one log-sum-exp per thread");
    auto row0_of = [&](const Tile1 &tl) __attribute__((always_inline)) {
        return min(win_start(tl.t0, T, ks), inv_lo(tl.t0, ks));
    };
    auto prefetch = [&](const Tile1 &tl) __attribute__((always_inline)) {
        const int ra = row0_of(tl);
        qst.fetch(seq(a.q, tl), a.q.sw, ra, T, dlim);
        kst.fetch(seq(a.k, tl), a.k.sw, ra, T, dlim);
        vst.fetch(seq(a.v, tl), a.v.sw, ra, T, dlim);
        gst.fetch(seq(a.d_o, tl), a.d_o.sw, ra, T, dlim);
        ost.fetch(seq(a.o, tl), a.o.sw, ra, T, dlim);
        const int64_t sq0 = ((int64_t)tl.bb * s.N + tl.nn) * T;
        lse_st = a.lse[sq0 + min(ra + min((int)threadIdx.x, NR - 1), T - 1)];
    };
    Tile1 cur = tile1_of(sc.t, tiles_t, s.N);
    prefetch(cur);
    auto commit = [&]() __attribute__((always_inline)) {
        qst.commit(lds_q, dlim);
        gst.commit(lds_g, dlim);
        kst.commit(lds_k, dlim);
        vst.commit(lds_v, dlim);
#pragma unroll
        for (int i = 0; i < St::NL; i++) {
            const float d = group_sum<CPR>(dot8<BF>(gst.v[i], ost.v[i]));
            const int r = (int)threadIdx.x / CPR + i * St::RPP;
            if (r < NR && threadIdx.x % CPR == 0) lds_stat[r].y = d;
        }
        if (threadIdx.x < NR) lds_stat[threadIdx.x].x = lse_st * kLog2e;
    };
    if constexpr (FULL) commit();
    for (;;) {
        if constexpr (!FULL) commit();
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        Tile1 nxt = cur;
        if (more) {
            nxt = tile1_of(tn, tiles_t, s.N);
            prefetch(nxt);
        } else {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last tile (nothing is loaded, and the explicit wait says so to the compiler)
        }
        const int ra = row0_of(cur);
        const int w0 = cur.t0 + wave * 16;
        if (FULL || w0 < T) {
            const bool live = w0 + n < T;
            const int pt = min(w0 + n, T - 1);  // this lane's position, as query and as key
            const int64_t goff = a.grad_at(cur.bb, cur.nn, 0, pt);
            const int own = pt - ra;
            {
                // ---- dQ: the wave's keys are the 16 + k - 1 positions from the window start
                // of its first query on
                const int sr0 = win_start(w0, T, ks);
                const int orow = sr0 - ra, dd = win_start(pt, T, ks) - sr0;
                auto trow = [&](int tk) __attribute__((always_inline)) {
                    return tk < ntok ? orow + tk : (int)NR;
                };
                s16x8 qreg[G::DS], greg[G::DS];
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    qreg[ds] = *reinterpret_cast<const s16x8 *>(lds_q + own * G::PITCH + g * 8 + ds * 32);
                    greg[ds] = *reinterpret_cast<const s16x8 *>(lds_g + own * G::PITCH + g * 8 + ds * 32);
                }
                const float2 mine = lds_stat[own];
                s16x8 dsb[G::KSTEPS];
#pragma unroll
                for (int mt = 0; mt < G::MT; mt++) {
                    const int row = trow(mt * 16 + n);
                    const short *kp = lds_k + row * G::PITCH + g * 8, *vp = lds_v + row * G::PITCH + g * 8;
                    f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ds = 0; ds < G::DS; ds++) {
                        cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(kp + ds * 32), qreg[ds], cs);
                        cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(vp + ds * 32), greg[ds], cp);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int tk = mt * 16 + g * 4 + i;
                        const bool ok = (unsigned)(tk - dd) < (unsigned)ks;
                        const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - mine.x : -INFINITY);
                        dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - mine.y));
                    }
                }
                f32x4 dq[G::DT];
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int kk = 0; kk < G::KSTEPS; kk++) {
                    const short *kp[2];
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        kp[h] = lds_k + trow(kk * 32 + h * 16 + g * 4 + (n >> 2)) * G::PITCH + (n & 3) * (D / 4);
#pragma unroll
                    for (int mt = 0; mt < G::DT; mt++)
                        dq[mt] = mfma16<BF>(cat(lds_read_tr(kp[0] + mt * 4), lds_read_tr(kp[1] + mt * 4)),
                                            dsb[kk], dq[mt]);
                }
                store_token<BF, D, D == 64 && !kNarrow, FULL>(static_cast<short *>(a.dq) + goff, g, dq, s.scale, live, dlim);
            }
            {
                // ---- dK, dV: the queries that attend to any of the wave's 16 keys, 32 at a time
                s16x8 kreg[G::DS], vreg[G::DS];
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    kreg[ds] = *reinterpret_cast<const s16x8 *>(lds_k + own * G::PITCH + g * 8 + ds * 32);
                    vreg[ds] = *reinterpret_cast<const s16x8 *>(lds_v + own * G::PITCH + g * 8 + ds * 32);
                }
                f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                    dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
                const int wa = inv_lo(w0, ks), wb = inv_hi(min(w0 + 16, T) - 1, T, ks);
                const int nq = wb - wa, r0 = wa - ra;
                auto row_of = [&](int qi) __attribute__((always_inline)) {
                    return qi < nq ? r0 + qi : (int)NR;
                };
                for (int q0 = 0; q0 < nq; q0 += 32) {
                    s16x8 pb, dsb;
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++) {
                        const int row = row_of(q0 + m2 * 16 + n);
                        const short *qp = lds_q + row * G::PITCH + g * 8, *gp = lds_g + row * G::PITCH + g * 8;
                        f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ds = 0; ds < G::DS; ds++) {
                            cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(qp + ds * 32), kreg[ds], cs);
                            cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(gp + ds * 32), vreg[ds], cp);
                        }
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int qi = q0 + m2 * 16 + g * 4 + i;
                            const float2 st = lds_stat[row_of(qi)];
                            const bool ok = (qi < nq) &
                                            ((unsigned)(pt - win_start(wa + qi, T, ks)) < (unsigned)ks);
                            const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
                            pb[m2 * 4 + i] = cvt16<BF>(p);
                            dsb[m2 * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                        }
                    }
                    const short *qt[2], *gt[2];
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int row = row_of(q0 + h * 16 + g * 4 + (n >> 2));
                        qt[h] = lds_q + row * G::PITCH + (n & 3) * (D / 4);
                        gt[h] = lds_g + row * G::PITCH + (n & 3) * (D / 4);
                    }
#pragma unroll
                    for (int mt = 0; mt < G::DT; mt++) {
                        dv[mt] = mfma16<BF>(cat(lds_read_tr(gt[0] + mt * 4), lds_read_tr(gt[1] + mt * 4)), pb, dv[mt]);
                        dk[mt] = mfma16<BF>(cat(lds_read_tr(qt[0] + mt * 4), lds_read_tr(qt[1] + mt * 4)), dsb, dk[mt]);
                    }
                }
                store_token<BF, D, D == 64 && !kNarrow, FULL>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, live, dlim);
                store_token<BF, D, D == 64 && !kNarrow, FULL>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, live, dlim);
            }
        }
        if (!more) {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            break;
        }
        __syncthreads();
        if constexpr (FULL) commit();
        cur = nxt;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dispatch
template <bool BF, int D, int NKP>
int fwd1d_launch(const FwdArgs &a, hipStream_t st) {
    const int tiles_t = (a.s.W + 63) / 64;
    const int64_t nt = (int64_t)a.s.B * a.s.N * tiles_t;
    const int grid = persistent_grid<fwd1d_mfma<BF, D, NKP>>(nt);
    {
        ProfScope prof(ENATTEN_KERNEL_FWD, "fwd1d_mfma", st);
        hipLaunchKernelGGL((fwd1d_mfma<BF, D, NKP>), dim3(grid), dim3(256), 0, st, a, tiles_t, (int)nt);
    }
    return check_launch("enatten1d_fwd");
}

template <bool BF, int D, int NKP>
int bwd1d_fused_launch(const BwdArgs &a, hipStream_t st) {
    const int tiles_t = (a.s.W + 63) / 64;
    const int64_t nt = (int64_t)a.s.B * a.s.N * tiles_t;
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_FUSED, "bwd1d_fused_mfma", st);
        const int grid = persistent_grid<bwd1d_fused_mfma<BF, D, NKP>>(nt);
        constexpr bool kFull = !kNarrow && D == 128;
        if (kFull && a.s.W % 64 == 0)
            hipLaunchKernelGGL((bwd1d_fused_mfma<BF, D, NKP, kFull>), dim3(grid), dim3(256), 0, st, a, tiles_t,
                               (int)nt);
        else
            hipLaunchKernelGGL((bwd1d_fused_mfma<BF, D, NKP>), dim3(grid), dim3(256), 0, st, a, tiles_t, (int)nt);
    }
    return check_launch("enatten1d_bwd");
}

template <bool BF, int D, int NKP>
int bwd1d_launch(const BwdArgs &a, hipStream_t st) {
    const int tiles_t = (a.s.W + 63) / 64;
    const int64_t nt = (int64_t)a.s.B * a.s.N * tiles_t;
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd1d_dq_mfma", st);
        hipLaunchKernelGGL((bwd1d_dq_mfma<BF, D, NKP>), dim3(persistent_grid<bwd1d_dq_mfma<BF, D, NKP>>(nt)),
                           dim3(256), 0, st, a, tiles_t, (int)nt);
    }
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd1d_dkdv_mfma", st);
        hipLaunchKernelGGL((bwd1d_dkdv_mfma<BF, D, NKP>),
                           dim3(persistent_grid<bwd1d_dkdv_mfma<BF, D, NKP>>(nt)), dim3(256), 0, st, a,
                           tiles_t, (int)nt);
    }
    return check_launch("enatten1d_bwd");
}

// A head dim that is a multiple of 8 runs on the kernels built for the next of 32, 64, 128.
constexpr int built_dim1(int D) { return D <= 32 ? 32 : D <= 64 ? 64 : 128; }
#define ENATTEN_1D_BY_D(FN, BF, NKP, ARGS, ST)                     \
    switch (built_dim1((ARGS).s.D)) {                              \
        case 32: return FN<BF, 32, NKP>(ARGS, ST);                 \
        case 64: return FN<BF, 64, NKP>(ARGS, ST);                 \
        case 128: return FN<BF, 128, NKP>(ARGS, ST);               \
    }
#define ENATTEN_1D(FN, ARGS, DTYPE, ST)                            \
    if ((DTYPE) == ENATTEN_BF16) {                                 \
        if ((ARGS).s.kw <= 17) { ENATTEN_1D_BY_D(FN, true, 32, ARGS, ST) }  \
        else { ENATTEN_1D_BY_D(FN, true, 64, ARGS, ST) }           \
    } else {                                                       \
        if ((ARGS).s.kw <= 17) { ENATTEN_1D_BY_D(FN, false, 32, ARGS, ST) } \
        else { ENATTEN_1D_BY_D(FN, false, 64, ARGS, ST) }          \
    }

// rows read with 16-byte loads: aligned base, strides that are multiples of 8
// elements, a position stride small enough for a 24-bit multiply of byte offsets
bool layout1d_ok(const View &v) {
    return reinterpret_cast<uintptr_t>(v.ptr) % 16 == 0 && v.sb % 8 == 0 && v.sn % 8 == 0 &&
           v.sw % 8 == 0 && v.sw < (1 << 22);
}

int fwd1d_dispatch(const FwdArgs &a, int dtype, hipStream_t st) {
    if (!layout1d_ok(a.q) || !layout1d_ok(a.k) || !layout1d_ok(a.v) || !layout1d_ok(a.o))
        return launch_fwd_simt(a, dtype, st);
    ENATTEN_1D(fwd1d_launch, a, dtype, st)
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kw);
    return ENATTEN_EUNSUPPORTED;
}

// One-pass backward where it was measured faster than the two passes: every head_dim for
// kernel_size <= 17, head_dim <= 64 beyond (at head_dim 128 the 136 staged rows of four
// tensors fill LDS and the two are level).
bool fused1d_supported(const BwdArgs &a) {
    return (a.s.kw <= 17 || a.s.D <= 64) && layout1d_ok(a.o);
}

int bwd1d_dispatch(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    auto al = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (!layout1d_ok(a.q) || !layout1d_ok(a.k) || !layout1d_ok(a.v) || !layout1d_ok(a.d_o) ||
        !al(a.dq) || !al(a.dk) || !al(a.dv) || a.gsb % 8 != 0 || a.gsn % 8 != 0 || a.gsw % 8 != 0)
        return launch_bwd_simt(a, dtype, st);
    if (!split_forced(path) && fused1d_supported(a)) {
        ENATTEN_1D(bwd1d_fused_launch, a, dtype, st)
    }
    ENATTEN_1D(bwd1d_launch, a, dtype, st)
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kw);
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace
}  // namespace enatten
