// Matrix-core kernels for float32 2D neighborhood attention on gfx950.
//
// float32 tensors need more than float32 logits: with unscaled q.k of magnitude ~50
// (the reference's benchmark inputs, e_natten/triton.py:280 applies no scale) a float32
// dot product is good to ~1e-5, which exp() turns into a relative error of the
// probabilities and ~1e-4 absolute error of dQ and dK.  So the logits are formed with
// the float64 matrix instruction v_mfma_f64_16x16x4_f64 and every other product (P.V,
// dO.V, dS.K, P^T.dO, dS^T.Q) with the float32 one, v_mfma_f32_16x16x4_f32: true
// float32 products, no reduced-precision operands anywhere.
//
// Geometry as in the 16-bit kernels: a workgroup of four waves owns an 8x8 tile of
// pixels, a wave a 4x4 block; the wave's 16 pixels are the N dimension of the matrix
// instructions, the (4+k-1)^2 pixels of its halo the token dimension.  One tensor's
// halo at a time is staged in LDS (float32 rows of D + 4 floats), so two workgroups
// share a CU; the other tensor's halo travels from HBM into registers meanwhile.
//
// Token numbering.  The float64 instruction leaves lane (n, g) with rows g, g+4, g+8,
// g+12 of a 16-row tile, the float32 one with rows 4g .. 4g+3.  Token t of a 16-token
// tile is the pixel (t & 3, t >> 2) of a 4x4 patch of the halo when the halo side is a
// multiple of 4 (kernel_size 5, 9, 13), so the four tokens of one reduction step of
// the second products (g = 0..3) sit in four different halo rows, 12 LDS rows apart,
// and their operand reads fall into disjoint banks; for other kernel sizes tokens are
// numbered row by row.  Where a float32 product has to line up with the float64 one
// (dP with P), its operand rows are fetched in the transposed order t -> 4(t&3) + t>>2.
//
// Backward.  The dQ pass recomputes the logits once (float64), forms P, dP, dS and dQ,
// and leaves P and dS of every (query, window position) in the workspace, k*k float32
// each per query.  The dK/dV pass then has no logits, masks or exponentials left: per
// key tile it walks the queries that attend to the tile (e_natten/pytorch.py:13-23,
// :261-270) and accumulates dV = P^T dO and dK = dS^T Q with the matrix instruction,
// P and dS gathered from the workspace (zero where a query does not attend a key).
// No atomics; results are bit-reproducible.
//
// Per-query math: e_natten/triton.py:242-302 (forward), :383-423 (backward).

#include "na2d_mfma.h"

namespace enatten {
namespace {

typedef double f64x4 __attribute__((ext_vector_type(4)));

template <int D, int KS>
struct Geo32 {
    static constexpr int HR = 8 + KS - 1, HC = HR;   // halo of the 8x8 tile
    static constexpr int SW = 4 + KS - 1;            // halo side of a wave's 4x4 block
    static constexpr bool PATCH = SW % 4 == 0;
    static constexpr int NK = SW * SW;
    static constexpr int NKP = (NK + 15) / 16 * 16;
    static constexpr int MT = NKP / 16;              // 16-token tiles
    static constexpr int KK = KS * KS;
    static constexpr int PITCH = D + 4;              // floats between LDS rows
    static constexpr int ROWS = HR * HC + 1;         // + an all-zero row for padding tokens
    static constexpr int ZROW = HR * HC;
    static constexpr int CPR = D / 4;                // 16-byte chunks per row
    static constexpr int NCH = HR * HC * CPR;
    static constexpr int NL = (NCH + 255) / 256;     // chunks per thread
    static constexpr int DQ = D / 4;                 // channels per lane group in the first products
    static constexpr int DT = D / 16;                // 16-channel tiles of the outputs
    static constexpr size_t LDS_BYTES = (size_t)ROWS * PITCH * sizeof(float);
    // (row, column) inside the wave's halo of token t of tile mt; false: no such token
    static __device__ __forceinline__ bool tok_rc(int mt, int t, int &r, int &c) {
        if constexpr (PATCH) {
            constexpr int PR = SW / 4;
            r = 4 * (mt / PR) + (t & 3);
            c = 4 * (mt % PR) + (t >> 2);
            return true;
        } else {
            const int tk = mt * 16 + t;
            r = tk / SW;
            c = tk % SW;
            return tk < NK;
        }
    }
    static __device__ __forceinline__ int tok_row(int mt, int t, int orow, int ocol) {
        int r, c;
        return tok_rc(mt, t, r, c) ? (orow + r) * HC + ocol + c : (int)ZROW;
    }
};

// Whole-line stores (store32's LINES) where LDS admits two workgroups per CU: like the 16-bit
// kernels, those with one workgroup per CU (head_dim 128 at kernel_size 7) do not gain from them.
template <int D, int KS>
constexpr bool kLines32 = 2 * Geo32<D, KS>::LDS_BYTES <= 160 * 1024;

struct Regs32 {
    // the largest halo served: kernel_size 7 at head_dim 128 is 196 pixels x 32 chunks
    u32x4 v[25];
};

// One tensor's halo (origin (hr0, hc0), pixels at or beyond (rlim, clim) clamped) into
// registers, then into LDS.
template <int D, int KS>
__device__ __forceinline__ void fetch32(Regs32 &reg, const float *img, int64_t sh, int64_t sw,
                                        int hr0, int hc0, int rlim, int clim) {
    using G = Geo32<D, KS>;
    static_assert(G::NL <= 25, "staging registers");
    const char *base = reinterpret_cast<const char *>(img + hr0 * sh + hc0 * sw);
    const unsigned sh4 = (unsigned)sh * 4u, sw4 = (unsigned)sw * 4u;
    const int rmax = rlim - 1 - hr0, cmax = clim - 1 - hc0;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        int pix = (int)threadIdx.x / G::CPR + i * (256 / G::CPR);
        pix = pix < G::HR * G::HC ? pix : G::HR * G::HC - 1;
        const unsigned r = (unsigned)min(pix / G::HC, rmax), c = (unsigned)min(pix % G::HC, cmax);
        const unsigned off = __umul24(r, sh4) + __umul24(c, sw4) + ((unsigned)threadIdx.x % G::CPR) * 16u;
        reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off);
    }
}
// The same in PARTS slices, so that the loads can be issued a few at a time between
// matrix instructions (a wave that issues a whole halo at once is blocked for
// microseconds while the CU's memory queue takes the loads, and issues no matrix
// instruction meanwhile).
// TAIL: the last TAIL chunks of a thread are left out of the slices (part == PARTS loads them):
// a kernel that has no registers for the whole halo beside its arithmetic loads them when the
// arithmetic is over, instead of having the compiler spill freshly loaded chunks to scratch
// memory, each behind a wait for its load.
template <int D, int KS, int PARTS, int TAIL = 0>
__device__ __forceinline__ void fetch32_part(Regs32 &reg, const float *img, int64_t sh, int64_t sw,
                                             int hr0, int hc0, int rlim, int clim, int part) {
    using G = Geo32<D, KS>;
    static_assert(TAIL < G::NL, "the tail is a part of the halo");
    const char *base = reinterpret_cast<const char *>(img + hr0 * sh + hc0 * sw);
    const unsigned sh4 = (unsigned)sh * 4u, sw4 = (unsigned)sw * 4u;
    const int rmax = rlim - 1 - hr0, cmax = clim - 1 - hc0;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        if ((i >= G::NL - TAIL ? PARTS : i * PARTS / (G::NL - TAIL)) != part) continue;
        int pix = (int)threadIdx.x / G::CPR + i * (256 / G::CPR);
        pix = pix < G::HR * G::HC ? pix : G::HR * G::HC - 1;
        const unsigned r = (unsigned)min(pix / G::HC, rmax), c = (unsigned)min(pix % G::HC, cmax);
        const unsigned off = __umul24(r, sh4) + __umul24(c, sw4) + ((unsigned)threadIdx.x % G::CPR) * 16u;
        reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off);
    }
}
template <int D, int KS>
__device__ __forceinline__ void commit32(float *lds, const Regs32 &reg) {
    using G = Geo32<D, KS>;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        const int pix = (int)threadIdx.x / G::CPR + i * (256 / G::CPR);
        if (pix < G::HR * G::HC)
            *reinterpret_cast<u32x4 *>(lds + pix * G::PITCH + ((int)threadIdx.x % G::CPR) * 4) = reg.v[i];
    }
}

// exp(x) for x <= 0 with a float64 argument through the hardware 2^y: the float32
// rounding of y = x * log2(e) is put back to first order, 2^(hi + lo) = 2^hi (1 + lo ln 2).
__device__ __forceinline__ float exp_neg64(double x) {
    const double y = fmax(x * 1.4426950408889634, -200.0);  // also maps -inf to an exact 0
    const float hi = (float)y;
    const float lo = (float)(y - (double)hi);
    const float e = __builtin_amdgcn_exp2f(hi);
    return fmaf(e, lo * kLn2, e);
}

// XCD-aware tile of a workgroup: every XCD takes one contiguous run of tiles.
__device__ __forceinline__ int tile_of_block(int ntiles) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per = (ntiles + 7) >> 3;
    const int t = xcd * per + slot;
    return (slot < per && t < ntiles) ? t : -1;
}

// logits^T [token][query] of the wave's halo in float64: acc[mt][e] is token e*4 + g of
// tile mt for this lane's query.  `qf` holds the query's channels g*D/4 ..
// The MT token tiles advance together, four channels at a time: MT independent
// accumulator chains, and a query channel is converted to float64 once for all of them.
// `hook(j)` runs before the instructions of channel group j of D/16 (used to issue
// global loads a few at a time).
template <int D, int KS, typename Hook>
__device__ __forceinline__ void logits64(const float *lds_k, const float *qf, int orow, int ocol,
                                         int n, int g, f64x4 *acc, Hook hook) {
    using G = Geo32<D, KS>;
    const float *kp[G::MT];
#pragma unroll
    for (int mt = 0; mt < G::MT; mt++) {
        kp[mt] = lds_k + G::tok_row(mt, n, orow, ocol) * G::PITCH + g * G::DQ;
        acc[mt] = f64x4{0.0, 0.0, 0.0, 0.0};
    }
#pragma unroll
    for (int j = 0; j < G::DQ / 4; j++) {
        __builtin_amdgcn_sched_barrier(0);
        hook(j);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 k4[G::MT];
#pragma unroll
        for (int mt = 0; mt < G::MT; mt++) k4[mt] = *reinterpret_cast<const f32x4 *>(kp[mt] + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const double qd = (double)qf[4 * j + e];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
                acc[mt] = __builtin_amdgcn_mfma_f64_16x16x4f64((double)k4[mt][e], qd, acc[mt], 0, 0, 0);
        }
    }
}

// out^T [channel][query] += X^T w over the wave's halo tokens, X rows from LDS:
// acc[m][e] is channel 16 m + 4 g + e of this lane's query.  w[mt][e] belongs to token
// e*4 + g of tile mt (the layout logits64 leaves).
// `hook(step)` runs before the instructions of reduction step `step` of MT * 4.
template <int D, int KS, typename Hook>
__device__ __forceinline__ void second32(const float *lds_x, const f32x4 *w, int orow, int ocol,
                                         int n, int g, f32x4 *acc, Hook hook) {
    using G = Geo32<D, KS>;
#pragma unroll
    for (int m = 0; m < G::DT; m++) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    // One reduction step is DT matrix instructions that share w[mt][e]; their DT operands
    // are read from LDS a step ahead, so the instructions never wait for LDS.
    constexpr int STEPS = G::MT * 4;
    float x[2][G::DT];
    auto fetch = [&](int step, float *dst) __attribute__((always_inline)) {
        const float *xp = lds_x + G::tok_row(step >> 2, (step & 3) * 4 + g, orow, ocol) * G::PITCH + n;
#pragma unroll
        for (int m = 0; m < G::DT; m++) dst[m] = xp[16 * m];
    };
    fetch(0, x[0]);
#pragma unroll
    for (int step = 0; step < STEPS; step++) {
        if (step + 1 < STEPS) fetch(step + 1, x[(step + 1) & 1]);
        hook(step);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < G::DT; m++)
            acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[step & 1][m], w[step >> 2][step & 3], acc[m], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Stores one token's D channels.  Piece m of lane group g is channels 16m + 4g .. +3, so the
// four lanes of a token would write 64 contiguous bytes per instruction: half a line, and
// non-temporal half lines reach memory in pieces (1.2-1.4x the bytes, at 3.1 TB/s against 5.3 for
// whole lines).  With LINES the lanes of tokens n and n^1 (adjacent lanes) exchange every other
// piece, and the eight lanes of the pair write one token's whole 128-byte line per instruction.
// Every lane of the wave must call this; `live`: this lane's token exists.
template <int D, bool LINES>
__device__ __forceinline__ void store32(float *token, int g, const f32x4 *acc, float mul, bool live) {
    if constexpr (LINES) {
        const bool odd = threadIdx.x & 1;
        auto xchg = [](unsigned x) __attribute__((always_inline)) {
            return (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true);
        };
        const uintptr_t own = reinterpret_cast<uintptr_t>(token);
        const uintptr_t nbr = (uintptr_t)xchg((unsigned)own) | ((uintptr_t)xchg((unsigned)(own >> 32)) << 32);
        // (as an offset from this lane's pointer, so that the stores stay global-memory instructions)
        float *other = reinterpret_cast<float *>(reinterpret_cast<char *>(token) + (ptrdiff_t)(nbr - own));
        const bool nlive = xchg(live ? 1u : 0u) != 0;
        float *tok_a = odd ? other : token, *tok_b = odd ? token : other;
        const bool live_a = odd ? nlive : live, live_b = odd ? live : nlive;
        const int off = (odd ? 16 : 0) + 4 * g;
#pragma unroll
        for (int k = 0; k < D / 32; k++) {
            const f32x4 lo = acc[2 * k] * mul, hi = acc[2 * k + 1] * mul;
            f32x4 sa, sb;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const float r = __uint_as_float(xchg(__float_as_uint(odd ? lo[c] : hi[c])));
                sa[c] = odd ? r : lo[c];
                sb[c] = odd ? hi[c] : r;
            }
            if (live_a) __builtin_nontemporal_store(sa, reinterpret_cast<f32x4 *>(tok_a + 32 * k + off));
            if (live_b) __builtin_nontemporal_store(sb, reinterpret_cast<f32x4 *>(tok_b + 32 * k + off));
        }
    } else {
        if (!live) return;
#pragma unroll
        for (int m = 0; m < D / 16; m++)
            __builtin_nontemporal_store(acc[m] * mul, reinterpret_cast<f32x4 *>(token + 16 * m + 4 * g));
    }
}

__device__ __forceinline__ const float *image32(const View &v, const Tile &tl) {
    return static_cast<const float *>(v.ptr) + tl.bb * v.sb + tl.nn * v.sn;
}

// this lane's share of one pixel's channels for the first products: channels
// g*D/4 .. (g+1)*D/4 - 1, as float32
template <int D>
__device__ __forceinline__ void load_quarter(const float *row, int g, float *out) {
#pragma unroll
    for (int j = 0; j < D / 16; j++) {
        const f32x4 x = *reinterpret_cast<const f32x4 *>(row + g * (D / 4) + 4 * j);
#pragma unroll
        for (int e = 0; e < 4; e++) out[4 * j + e] = x[e];
    }
}

// Is halo token (r, c) inside the window of the query whose window starts at (dr, dc)?
template <int KS>
__device__ __forceinline__ bool in_window(int r, int c, int dr, int dc) {
    return (unsigned)(r - dr) < (unsigned)KS && (unsigned)(c - dc) < (unsigned)KS;
}

// ------------------------------------------------------------------ forward
// S^T = K Q^T (float64), masked softmax, O^T = V^T P^T (float32); writes O and the
// log-sum-exp.  Persistent: K's halo is in LDS while the logits are formed and V's halo
// is loaded, a few loads between the matrix instructions of each token tile; then V's
// halo takes K's place, and the next tile's K is loaded between the instructions of P.V.
template <int D, int KS>
__global__ __launch_bounds__(256, 2) void fwd_mfma_f32(FwdArgs a, int tiles_r, int tiles_c, int ntiles) {
    using G = Geo32<D, KS>;
    constexpr int STEPS = G::MT * 4;
    __shared__ __attribute__((aligned(16))) float lds[G::ROWS * G::PITCH];
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    const Shape &s = a.s;
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    if (threadIdx.x < G::PITCH) lds[G::ZROW * G::PITCH + threadIdx.x] = 0.f;

    Tile cur = tile_of(sc.t, tiles_r, tiles_c, s.N);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    Regs32 st;
    float qf[G::DQ];
    fetch32<D, KS>(st, image32(a.k, cur), a.k.sh, a.k.sw, lq.hr0, lq.hc0, s.H, s.W);
    load_quarter<D>(image32(a.q, cur) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, qf);
    for (;;) {
        commit32<D, KS>(lds, st);
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        const Tile nxt = more ? tile_of(tn, tiles_r, tiles_c, s.N) : cur;
        const LaneQ lqn = lane_query<KS>(nxt, s, wave, n);
        const float *vimg = image32(a.v, cur), *kimg = image32(a.k, nxt);
        auto load_v = [&](int part) __attribute__((always_inline)) {
            fetch32_part<D, KS, G::DQ / 4>(st, vimg, a.v.sh, a.v.sw, lq.hr0, lq.hc0, s.H, s.W, part);
        };
        auto load_next = [&](int part) __attribute__((always_inline)) {
            if (more) {
                fetch32_part<D, KS, STEPS>(st, kimg, a.k.sh, a.k.sw, lqn.hr0, lqn.hc0, s.H, s.W, part);
                if (part == STEPS - 1)
                    load_quarter<D>(image32(a.q, nxt) + lqn.qr * a.q.sh + lqn.qc * a.q.sw, g, qf);
            }
        };

        f32x4 p[G::MT];
        float lse = 0.f, inv = 0.f;
        if (lq.wave_on) {
            f64x4 acc[G::MT];
            logits64<D, KS>(lds, qf, lq.orow, lq.ocol, n, g, acc, load_v);
            double mx = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    int r, c;
                    const bool ok = G::tok_rc(mt, e * 4 + g, r, c) && in_window<KS>(r, c, lq.dr, lq.dc);
                    acc[mt][e] = ok ? acc[mt][e] * (double)s.scale : -INFINITY;
                    mx = fmax(mx, acc[mt][e]);
                }
            mx = fmax(mx, __shfl_xor(mx, 16, 64));
            mx = fmax(mx, __shfl_xor(mx, 32, 64));
            float sum = 0.f;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    p[mt][e] = exp_neg64(acc[mt][e] - mx);
                    sum += p[mt][e];
                }
            sum = col_sum(sum);
            inv = 1.f / sum;
            lse = (float)(mx + (double)logf(sum));
        } else {
#pragma unroll
            for (int part = 0; part < G::DQ / 4; part++) load_v(part);
        }
        __syncthreads();  // every wave is done with K
        commit32<D, KS>(lds, st);
        __syncthreads();
        if (lq.wave_on) {
            f32x4 o[G::DT];
            second32<D, KS>(lds, p, lq.orow, lq.ocol, n, g, o, load_next);
            float *op = const_cast<float *>(image32(a.o, cur)) + lq.qr * a.o.sh + lq.qc * a.o.sw;
            store32<D, kLines32<D, KS>>(op, g, o, inv, lq.live);
            if (lq.live && a.lse && g == 0) a.lse[lq.tok] = lse;
        } else {
#pragma unroll
            for (int part = 0; part < STEPS; part++) load_next(part);
        }
        if (!more) break;
        __syncthreads();  // every wave is done with V
        cur = nxt;
        lq = lqn;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dQ (+ P, dS)
// dP^T = V dO^T (float32) on V's halo, then K's halo into the same rows: logits in
// float64, P renormalised over the window (which removes the rounding of the stored
// log-sum-exp), delta = sum_j P_j dP_j, dS = P (dP - delta), dQ^T = K^T dS^T.  P and dS
// go to the workspace, k*k values per query in window order, for the dK/dV pass.
// Persistent like the forward: K is loaded between the instructions of dP, the next
// tile's V between those of dQ.
// Chunks of a halo that the dQ pass loads behind its arithmetic (fetch32_part's TAIL), where it
// would spill otherwise.  B4 N4 128x128 d128 k5: 84 -> 12 bytes of scratch per lane and
// 261 -> 231 us; B4 N8 96x96 d32 k7: 76 -> 0 bytes, 194 -> 164 us; d64 k7: 288 -> 96 bytes,
// 319 -> 273 us (the whole halo behind the arithmetic: its float64 logits of 13 token tiles
// leave no registers for any of it).
template <int D, int KS>
constexpr int kDqTail = D == 128 && KS == 5 ? 5 : D == 32 && KS == 7 ? 5 : D == 64 && KS == 7 ? 12 : 0;

template <int D, int KS>
__global__ __launch_bounds__(256, 2) void bwd_dq_mfma_f32(BwdArgs a, float *ws_p, float *ws_ds,
                                                          int tiles_r, int tiles_c, int ntiles) {
    using G = Geo32<D, KS>;
    constexpr int STEPS = G::MT * 4;
    __shared__ __attribute__((aligned(16))) float lds[G::ROWS * G::PITCH];
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    const Shape &s = a.s;
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    if (threadIdx.x < G::PITCH) lds[G::ZROW * G::PITCH + threadIdx.x] = 0.f;

    Tile cur = tile_of(sc.t, tiles_r, tiles_c, s.N);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    Regs32 st;
    float go[G::DQ];
    fetch32<D, KS>(st, image32(a.v, cur), a.v.sh, a.v.sw, lq.hr0, lq.hc0, s.H, s.W);
    load_quarter<D>(image32(a.d_o, cur) + lq.qr * a.d_o.sh + lq.qc * a.d_o.sw, g, go);
    for (;;) {
        commit32<D, KS>(lds, st);
        __syncthreads();
        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        const Tile nxt = more ? tile_of(tn, tiles_r, tiles_c, s.N) : cur;
        const LaneQ lqn = lane_query<KS>(nxt, s, wave, n);
        const float *kimg = image32(a.k, cur), *vimg = image32(a.v, nxt);
        // this tile's q and log-sum-exp arrive while dP is formed (their registers are
        // free until then: dO's are needed first, q's afterwards)
        float qf[G::DQ];
        float lse_f = 0.f;
        auto load_k = [&](int part) __attribute__((always_inline)) {
            fetch32_part<D, KS, G::MT, kDqTail<D, KS>>(st, kimg, a.k.sh, a.k.sw, lq.hr0, lq.hc0, s.H, s.W, part);
            if (part == G::MT - 1) {
                load_quarter<D>(image32(a.q, cur) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, qf);
                lse_f = a.lse[lq.tok];
            }
        };

        // dP^T: the operand rows are fetched in the transposed order, so that accumulator
        // element e of lane group g is token e*4 + g like in the float64 product
        f32x4 dp[G::MT];
        if (lq.wave_on) {
            const int nt = ((n & 3) << 2) | (n >> 2);
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                __builtin_amdgcn_sched_barrier(0);
                load_k(mt);
                __builtin_amdgcn_sched_barrier(0);
                const float *vp = lds + G::tok_row(mt, nt, lq.orow, lq.ocol) * G::PITCH + g * G::DQ;
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int j = 0; j < G::DQ / 4; j++) {
                    const f32x4 v4 = *reinterpret_cast<const f32x4 *>(vp + 4 * j);
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        c = __builtin_amdgcn_mfma_f32_16x16x4f32(v4[e], go[4 * j + e], c, 0, 0, 0);
                }
                dp[mt] = c;
            }
        } else {
#pragma unroll
            for (int part = 0; part < G::MT; part++) load_k(part);
        }
        if constexpr (kDqTail<D, KS> > 0) load_k(G::MT);
        const double lse = (double)lse_f;
        __syncthreads();  // every wave is done with V
        commit32<D, KS>(lds, st);
        __syncthreads();
        auto load_next = [&](int part) __attribute__((always_inline)) {
            if (more) {
                fetch32_part<D, KS, STEPS, kDqTail<D, KS>>(st, vimg, a.v.sh, a.v.sw, lqn.hr0, lqn.hc0, s.H, s.W, part);
                if (part == STEPS - 1)
                    load_quarter<D>(image32(a.d_o, nxt) + lqn.qr * a.d_o.sh + lqn.qc * a.d_o.sw, g, go);
            }
        };
        if (lq.wave_on) {
            f32x4 ds[G::MT];
            {
                f64x4 acc[G::MT];
                logits64<D, KS>(lds, qf, lq.orow, lq.ocol, n, g, acc, [](int) {});
                float z = 0.f;
#pragma unroll
                for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int r, c;
                        const bool ok = G::tok_rc(mt, e * 4 + g, r, c) && in_window<KS>(r, c, lq.dr, lq.dc);
                        ds[mt][e] = ok ? exp_neg64(fmin(acc[mt][e] * (double)s.scale - lse, 0.0)) : 0.f;
                        z += ds[mt][e];
                    }
                const float zinv = 1.f / col_sum(z);
                float dpart = 0.f;
#pragma unroll
                for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        ds[mt][e] *= zinv;                       // P
                        dpart = fmaf(ds[mt][e], dp[mt][e], dpart);
                    }
                const float delta = col_sum(dpart);
                float *pp = ws_p + lq.tok * G::KK, *dsp = ws_ds + lq.tok * G::KK;
#pragma unroll
                for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        int r, c;
                        const bool ok = G::tok_rc(mt, e * 4 + g, r, c) && in_window<KS>(r, c, lq.dr, lq.dc);
                        const float pv = ds[mt][e];
                        ds[mt][e] = pv * (dp[mt][e] - delta);    // dS
                        if (ok && lq.live) {
                            const int j = (r - lq.dr) * KS + (c - lq.dc);
                            pp[j] = pv;
                            dsp[j] = ds[mt][e];
                        }
                    }
            }
            f32x4 dq[G::DT];
            second32<D, KS>(lds, ds, lq.orow, lq.ocol, n, g, dq, load_next);
            store32<D, kLines32<D, KS>>(static_cast<float *>(a.dq) + lq.tok * D, g, dq, s.scale, lq.live);
        } else {
#pragma unroll
            for (int part = 0; part < STEPS; part++) load_next(part);
        }
        if constexpr (kDqTail<D, KS> > 0) load_next(STEPS);
        if (!more) break;
        __syncthreads();  // every wave is done with K
        cur = nxt;
        lq = lqn;
        sc.t = tn;
    }
}

// ------------------------------------------------------------------ dK or dV
// Key-centric: the workgroup owns 8x8 keys, a wave 4x4 of them (the N dimension).  The
// queries that attend to any key of the tile form a rectangle (the union of the keys'
// inverse neighbourhoods, e_natten/pytorch.py:13-23), walked in blocks of at most
// (8+k-1)^2 queries whose X rows (dO for dV, Q for dK) are staged in LDS.  One
// reduction step takes the four queries (row r .. r+3, column c) of the wave's part of
// the block: their LDS rows are a halo row apart, so the operand reads fall into
// disjoint banks.  The weights W (P for dV, dS for dK) come from the workspace; a query
// that does not attend to a key contributes an exact zero.
template <int D, int KS>
__global__ __launch_bounds__(256, 2) void bwd_dkdv_mfma_f32(BwdArgs a, View x, const float *ws_w,
                                                            float *out, float mul, int tiles_r,
                                                            int tiles_c, int ntiles) {
    using G = Geo32<D, KS>;
    constexpr int NRG = (G::SW + KS / 2 + 3) / 4;   // groups of 4 query rows a wave can meet in a block
    constexpr int NC = G::SW + KS / 2;              // query columns likewise
    __shared__ __attribute__((aligned(16))) float lds[G::ROWS * G::PITCH];
    const int t = tile_of_block(ntiles);
    if (t < 0) return;
    const Shape &s = a.s;
    const Tile tl = tile_of(t, tiles_r, tiles_c, s.N);
    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    // the tile's and the wave's keys, and the queries that attend to them
    const int wr0 = tl.r0 + (wave >> 1) * 4, wc0 = tl.c0 + (wave & 1) * 4;
    const bool wave_on = wr0 < s.H && wc0 < s.W;
    const int kr = min(wr0 + (n >> 2), s.H - 1), kc = min(wc0 + (n & 3), s.W - 1);
    const bool live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
    const int qa = inv_lo(tl.r0, KS), qb = inv_hi(min(tl.r0 + 8, s.H) - 1, s.H, KS);
    const int ca = inv_lo(tl.c0, KS), cb = inv_hi(min(tl.c0 + 8, s.W) - 1, s.W, KS);
    const int wqa = inv_lo(min(wr0, s.H - 1), KS), wqb = inv_hi(min(wr0 + 4, s.H) - 1, s.H, KS);
    const int wca = inv_lo(min(wc0, s.W - 1), KS), wcb = inv_hi(min(wc0 + 4, s.W) - 1, s.W, KS);
    const float *ximg = image32(x, tl);
    const int64_t img_tok = ((int64_t)tl.bb * s.N + tl.nn) * s.H * (int64_t)s.W;

    f32x4 acc[G::DT];
#pragma unroll
    for (int m = 0; m < G::DT; m++) acc[m] = f32x4{0.f, 0.f, 0.f, 0.f};
    Regs32 st;
    for (int br = qa; br < qb; br += G::HR) {
        for (int bc = ca; bc < cb; bc += G::HC) {
            fetch32<D, KS>(st, ximg, x.sh, x.sw, br, bc, qb, cb);
            // this wave's queries inside the block
            const int ra = max(wqa, br), rb = min(wqb, br + G::HR);
            const int cc = max(wca, bc), cd = min(wcb, bc + G::HC);
            // weights of the block's reduction steps: query (ra + 4 rg + g, cc + c), this
            // lane's key; zero if the query is outside the wave's part or does not attend
            float w[NRG * NC];
#pragma unroll
            for (int rg = 0; rg < NRG; rg++)
#pragma unroll
                for (int c = 0; c < NC; c++) {
                    const int qr = ra + 4 * rg + g, qc = cc + c;
                    const int pr = kr - win_start(min(qr, s.H - 1), s.H, KS);
                    const int pc = kc - win_start(min(qc, s.W - 1), s.W, KS);
                    const bool ok = wave_on && qr < rb && qc < cd && (unsigned)pr < (unsigned)KS &&
                                    (unsigned)pc < (unsigned)KS;
                    w[rg * NC + c] = ok ? ws_w[(img_tok + (int64_t)qr * s.W + qc) * G::KK + pr * KS + pc] : 0.f;
                }
            __syncthreads();  // the previous block's rows are no longer read
            commit32<D, KS>(lds, st);
            __syncthreads();
            if (wave_on) {
                // A step's DT operands are read from LDS a step ahead of the matrix
                // instructions that use them.
                float x[2][G::DT];
                auto fetch = [&](int rg, int c, float *dst) __attribute__((always_inline)) {
                    // LDS row of this lane group's query row in the block (clamped: the
                    // weight of a row or column past the end is zero)
                    const int lrow = min(min(ra + 4 * rg + g, qb - 1) - br, G::HR - 1);
                    const int lcol = min(cc + c - bc, G::HC - 1);
                    const float *xp = lds + (lrow * G::HC + lcol) * G::PITCH + n;
#pragma unroll
                    for (int m = 0; m < G::DT; m++) dst[m] = xp[16 * m];
                };
                fetch(0, 0, x[0]);
#pragma unroll
                for (int rg = 0; rg < NRG; rg++) {
                    if (ra + 4 * rg >= rb) break;
#pragma unroll
                    for (int c = 0; c < NC; c++) {
                        const int step = rg * NC + c;
                        // the step after this one (it may lie past the end of the wave's
                        // part of the block: then its weight is zero or it is not run)
                        if (c + 1 < NC) fetch(rg, c + 1, x[(step + 1) & 1]);
                        else if (rg + 1 < NRG) fetch(rg + 1, 0, x[(step + 1) & 1]);
                        __builtin_amdgcn_sched_barrier(0);
                        if (cc + c < cd) {
#pragma unroll
                            for (int m = 0; m < G::DT; m++)
                                acc[m] = __builtin_amdgcn_mfma_f32_16x16x4f32(x[step & 1][m], w[step],
                                                                              acc[m], 0, 0, 0);
                        }
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    }
    if (!wave_on) return;
    const int64_t tok = img_tok + (int64_t)kr * s.W + kc;
    store32<D, kLines32<D, KS>>(out + tok * D, g, acc, mul, live);
}

// ------------------------------------------------------------------ dispatch
template <int D, int KS>
int fwd32_launch(const FwdArgs &a, hipStream_t st) {
    const int tiles_r = (a.s.H + 7) / 8, tiles_c = (a.s.W + 7) / 8;
    const int64_t nt = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
    const int grid = persistent_grid<fwd_mfma_f32<D, KS>>(nt);
    {
        ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_mfma_f32", st);
        hipLaunchKernelGGL((fwd_mfma_f32<D, KS>), dim3(grid), dim3(256), 0, st, a, tiles_r, tiles_c, (int)nt);
    }
    return check_launch("enatten2d_fwd");
}

template <int D, int KS>
int bwd32_launch(const BwdArgs &a, hipStream_t st) {
    const int tiles_r = (a.s.H + 7) / 8, tiles_c = (a.s.W + 7) / 8;
    const int64_t nt = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
    const int grid = (int)((nt + 7) / 8 * 8);
    const int64_t queries = (int64_t)a.s.B * a.s.N * a.s.H * a.s.W;
    float *ws_p = a.delta, *ws_ds = a.delta + queries * KS * KS;
    {
        ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_mfma_f32", st);
        hipLaunchKernelGGL((bwd_dq_mfma_f32<D, KS>), dim3(persistent_grid<bwd_dq_mfma_f32<D, KS>>(nt)),
                           dim3(256), 0, st, a, ws_p, ws_ds, tiles_r, tiles_c, (int)nt);
    }
    {
        // dV = P^T dO, then dK = dS^T Q: the same kernel on the other pair of operands
        ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd_dkdv_mfma_f32", st);
        hipLaunchKernelGGL((bwd_dkdv_mfma_f32<D, KS>), dim3(grid), dim3(256), 0, st, a, a.d_o, ws_p,
                           static_cast<float *>(a.dv), 1.f, tiles_r, tiles_c, (int)nt);
        hipLaunchKernelGGL((bwd_dkdv_mfma_f32<D, KS>), dim3(grid), dim3(256), 0, st, a, a.q, ws_ds,
                           static_cast<float *>(a.dk), a.s.scale, tiles_r, tiles_c, (int)nt);
    }
    return check_launch("enatten2d_bwd");
}

#define ENATTEN_F32_BY_KS(FN, D, ARGS, ST)                 \
    switch ((ARGS).s.kh) {                                 \
        case 3: return FN<D, 3>(ARGS, ST);                 \
        case 5: return FN<D, 5>(ARGS, ST);                 \
        case 7: return FN<D, 7>(ARGS, ST);                 \
    }
#define ENATTEN_F32_BY_D(FN, ARGS, ST)                     \
    switch ((ARGS).s.D) {                                  \
        case 32: ENATTEN_F32_BY_KS(FN, 32, ARGS, ST) break;   \
        case 64: ENATTEN_F32_BY_KS(FN, 64, ARGS, ST) break;   \
        case 128: ENATTEN_F32_BY_KS(FN, 128, ARGS, ST) break; \
    }

// 16-byte loads of float rows: aligned base, strides that are multiples of 4 floats,
// row and pixel strides small enough for 24-bit multiplies of byte offsets
bool layout32_ok(const View &v) {
    return reinterpret_cast<uintptr_t>(v.ptr) % 16 == 0 && v.sb % 4 == 0 && v.sn % 4 == 0 &&
           v.sh % 4 == 0 && v.sw % 4 == 0 && v.sh < (1 << 21) && v.sw < (1 << 21);
}

}  // namespace

// float32 tensors, head_dim 32 / 64 / 128, kernel_size 3 / 5 / 7
bool mfma_f32_supported(int D, int ks, int dtype) {
    return dtype == ENATTEN_F32 && (D == 32 || D == 64 || D == 128) && (ks == 3 || ks == 5 || ks == 7);
}

// float32 per query that the backward of these kernels needs in the workspace
size_t mfma_f32_workspace_floats(int ks) { return (size_t)2 * ks * ks; }

int launch_fwd_mfma_f32(const FwdArgs &a, hipStream_t st) {
    if (!layout32_ok(a.q) || !layout32_ok(a.k) || !layout32_ok(a.v) || !layout32_ok(a.o))
        return launch_fwd_simt(a, ENATTEN_F32, st);
    ENATTEN_F32_BY_D(fwd32_launch, a, st)
    set_error("no float32 matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

int launch_bwd_mfma_f32(const BwdArgs &a, hipStream_t st) {
    auto al = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (!layout32_ok(a.q) || !layout32_ok(a.k) || !layout32_ok(a.v) || !layout32_ok(a.d_o) ||
        !al(a.dq) || !al(a.dk) || !al(a.dv))
        return launch_bwd_simt(a, ENATTEN_F32, st);
    ENATTEN_F32_BY_D(bwd32_launch, a, st)
    set_error("no float32 matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace enatten
