// Matrix-core (MFMA) kernels for 2D neighborhood attention on gfx950.
//
// Geometry shared by all three kernels: a workgroup of four waves owns an 8x8
// tile of pixels of one (batch, head) image; each wave owns a 4x4 block of it.
// The 16 pixels of a wave are the N dimension of v_mfma_f32_16x16x32; the
// (4+k-1)^2 pixels of the block's halo are the other token dimension.  With the
// tokens of the halo as MFMA rows, every lane holds the logits of ONE query
// (column l%16) for several keys, so the softmax statistics need no transposes
// and the probabilities feed the second MFMA straight from the accumulators:
// the reduction index of the second product is enumerated in the order the
// accumulators hold it (slot e of lane group g <-> halo token 32*ks + 16*(e/4) +
// 4*g + e%4), and the other operand is fetched from LDS in that same order.
// That operand (V for O, K for dQ, dO/Q for dV/dK) is needed token-major while
// LDS holds it channel-major; ds_read_b64_tr_b16 does the transpose on the way
// out of LDS.  Output channels are likewise permuted (MFMA row g*4+i <-> channel
// g*D/4 + mt*4 + i) so that each lane ends up with D/4 contiguous channels of its
// query and writes them with 16-byte stores.
//
// Scheduling: the kernels are persistent.  Each workgroup walks a strided list
// of tiles and, while it computes one tile out of LDS, the global loads of the
// next tile's halo are already in flight into registers; they are written to LDS
// after the barrier that ends the current tile.  HBM latency is thus hidden
// behind compute even when LDS only admits one or two workgroups per CU.
//
// Forward follows e_natten/triton.py:242-302 per query (window start, mask,
// softmax, P.V); the log-sum-exp is kept for the backward.
//
// This file is compiled twice, by na2d_mfma.hip and by na2d_mfma_narrow.hip, each of
// which defines `enatten::(anonymous)::kNarrow` before including it.  false: the tensors'
// head dim IS the D a kernel is built for (32, 64, 128), and nothing below costs an
// instruction.  true: the head dim is any multiple of 8 up to D; the channels a tensor
// does not have are zero in LDS and in the operand registers and are left out of the
// stores (zero_row, HaloPlan::on, load_row_chunks, store_token in na2d_mfma.h).  One
// build serving both was measured 5-40% slower on the exact head dims (the predicates
// cost the large-halo kernels the registers they do not have).

#include <algorithm>

#include "na2d_mfma.h"

namespace enatten {
namespace {

// Whole-line stores (store_token's LINES) where a kernel runs at least two workgroups per CU
// on tensors of head_dim 128 or 64 itself (a token is then two aligned lines, or one).
// Measured, us, without -> with: d = 128 see store_token; d = 64 B4 N8 128x128 k5 forward 65.4 ->
// 61.4, dQ 67.8 -> 65.5, dK/dV 83.7 -> 76.1; B4 N4 256x256 k5 473 -> 427 per forward+backward;
// k7 284 -> 282; from k = 9 on the times do not change (343 -> 347, 281.4 -> 280.9 at k13: the
// kernels do not wait for their stores there), but the bytes do (dQ pass at d64 k13: 54.5 MB
// written for 34.6), so it is used at every kernel size.
// The dK/dV pass's inner tiles have no token outside the image, so their whole-line stores
// need no predicates (store_token's ALL), and without the branches that predicates put between
// the stores they pay at one workgroup per CU as well: dK/dV pass d128 k7 157.5 -> 154.6 us, k5
// 91.1 -> 88.7, d64 k5 82.1 -> 76.3, equal from k = 9 on.
template <int D>
constexpr bool kInnerLines = (D == 128 || D == 64) && !kNarrow;
template <int D, int KS, int WGS>
constexpr bool kLineStores = (D == 128 || D == 64) && !kNarrow && WGS >= 2;

// ------------------------------------------------------------------ forward
// ROLL: walk down the columns of an image and keep the halo rows that consecutive
// tiles share in LDS (see make_runs); otherwise a strided walk over row-major tiles
// with the whole halo staged per tile.
// FULL: the image sides are multiples of the tile sides, so every lane's pixel exists: no
// wave is switched off and no store is predicated.  The compiler then knows how many stores
// a tile issues, and the wait for the next tile's staged rows (older than those stores) does
// not wait for the stores as well.  With a branch around the stores, even a uniform one with
// an explicit wait on its other side, it falls back to waiting for everything outstanding
// (B4 N4 128x128 d128 k5: 58.8 -> 56.7 us, 256x256: 198.2 -> 189.3, d64 k5: 60.4 -> 58.5).
template <bool BF, int D, int KS, bool ROLL, int NW = 4, bool FULL = false>
__global__ __launch_bounds__((Geo<D, KS, NW>::NT), (Geo<D, KS, NW>::WAVES)) void fwd_mfma(FwdArgs a, int tiles_r, int tiles_c, int ntiles, Runs rp) {
    using G = Geo<D, KS, NW>;
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];

    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = ROLL ? make_runs(ntiles, blockIdx.x, gridDim.x, rp) : make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS, NW>(lds_k, dlim);
    zero_row<D, KS, NW>(lds_v, dlim);

    const int wave = FULL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;

    // registers that carry the next tile while the current one is computed
    const HaloPlan<D, KS, NW> plan = make_plan<D, KS, NW>(dlim);
    HaloRegs<D, KS, NW> kst, vst;
    s16x8 qnext[G::DS];
    // rows [y0, y0 + nr) of the halo are what LDS does not hold yet
    auto prefetch = [&](const Tile &tl, const LaneQ &lq, int y0, int nr) __attribute__((always_inline)) {
        if constexpr (ROLL) {
            halo_fetch_rows<D, KS>(kst, plan, image<short>(a.k, tl), a.k.sh, a.k.sw, y0, lq.hc0, nr, s.H, s.W);
            halo_fetch_rows<D, KS>(vst, plan, image<short>(a.v, tl), a.v.sh, a.v.sw, y0, lq.hc0, nr, s.H, s.W);
        } else {
            halo_fetch<D, KS>(kst, plan, image<short>(a.k, tl), a.k.sh, a.k.sw, lq.hr0, lq.hc0, s.H, s.W);
            halo_fetch<D, KS>(vst, plan, image<short>(a.v, tl), a.v.sh, a.v.sw, lq.hr0, lq.hc0, s.H, s.W);
        }
        load_row_chunks(qnext, image<short>(a.q, tl) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, dlim);
    };

    auto pick = [&](int t) __attribute__((always_inline)) {
        return ROLL ? tile_of_cm(t, tiles_r, tiles_c, s.N) : tile_of(t, tiles_r, tiles_c, s.N, G::TH);
    };
    Tile cur = pick(sc.t);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    int y0 = lq.hr0, nr = G::HR;
    prefetch(cur, lq, y0, nr);
    s16x8 qreg[G::DS];
    // FULL: the staged rows go to LDS at the END of a tile's pass through the loop, after its
    // stores, not at the top of the next: there the compiler has to merge the first pass (where
    // these loads are the youngest memory operations) with the later ones, and waits for
    // everything outstanding, the tile's own stores included.
    auto commit = [&]() __attribute__((always_inline)) {
        if constexpr (ROLL) {
            halo_commit_rows<D, KS>(lds_k, plan, kst, y0, nr);
            halo_commit_rows<D, KS>(lds_v, plan, vst, y0, nr);
        } else {
            halo_commit<D, KS>(lds_k, plan, kst);
            halo_commit<D, KS>(lds_v, plan, vst);
        }
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) qreg[ds] = qnext[ds];
    };
    if constexpr (FULL) commit();
    for (;;) {
        if constexpr (!FULL) commit();
        __syncthreads();

        const int tn = sched_peek(sc);
        const bool more = tn < sc.t_end;
        Tile nxt = cur;
        LaneQ lqn = lq;
        if (more) {
            nxt = pick(tn);
            lqn = lane_query<KS>(nxt, s, wave, n);
            // the tile below in the same image keeps the rows the two halos share
            const bool below = ROLL && nxt.bb == cur.bb && nxt.nn == cur.nn && nxt.c0 == cur.c0 &&
                               nxt.r0 > cur.r0 && lqn.hr0 < lq.hr0 + G::HR;
            y0 = below ? lq.hr0 + G::HR : lqn.hr0;
            nr = below ? lqn.hr0 - lq.hr0 : G::HR;
            prefetch(nxt, lqn, y0, nr);
        } else {
            // (the last tile of the walk: nothing is loaded, and the explicit wait says so to
            // the compiler, which does not know that this path leaves the loop below)
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        }
        const int rot = ROLL ? lq.hr0 % G::HR : 0;
        auto trow = [&](int tile, int x) __attribute__((always_inline)) {
            return ROLL ? G::token_row_rot(tile, x, lq.orow, lq.ocol, rot) : G::token_row(tile, x, lq.orow, lq.ocol);
        };

        if (FULL || lq.wave_on) {
            // logits^T [halo token][query], masked, in units of log2
            f32x4 acc[G::MT];
            float mx = -INFINITY;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const typename G::ARow kp = G::a_row(lds_k, trow(mt, n), g);
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++)
                    c = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(kp, ds)), qreg[ds], c);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, lq.dr, lq.dc);
                    c[i] = ok ? c[i] * sc2 : -INFINITY;
                    mx = fmaxf(mx, c[i]);
                }
                acc[mt] = c;
            }
            mx = col_max(mx);
            float sum = 0.f;
            s16x8 pb[G::KSTEPS];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float p = __builtin_amdgcn_exp2f(acc[mt][i] - mx);
                    sum += p;
                    pb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                }
            }
            sum = col_sum(sum);

            // O^T [channel][query] = V^T P^T over the halo tokens
            f32x4 o[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) o[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                typename G::TRow vp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    vp[h] = G::t_row(lds_v, trow(ks * 2 + h, g * 4 + (n >> 2)), n);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    o[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(vp[0], mt)), lds_read_tr(G::t_at(vp[1], mt))), pb[ks],
                        o[mt]);
            }

            store_token<BF, D, kLineStores<D, KS, G::WAVES>, FULL>(const_cast<short *>(image<short>(a.o, cur)) + lq.qr * a.o.sh + lq.qc * a.o.sw,
                               g, o, 1.f / sum, lq.live, dlim);
            // (FULL: all four lanes of a token write its log-sum-exp, the same value, so that
            // this store is not predicated either)
            if (a.lse && (FULL || (lq.live && g == 0)))
                a.lse[lq.tok] = (mx + __builtin_amdgcn_logf(sum)) * kLn2;
        }

        if (!more) {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // (as above: this path shares its last block with the other)
            break;
        }
        __syncthreads();  // every wave is done with this tile's LDS
        if constexpr (FULL) commit();
        cur = nxt;
        lq = lqn;
        sched_advance(sc, tn);
    }
}

// Two halos of an 8x8 tile fit LDS (the kernels that keep K and V, or Q and dO, side by side)
template <int D, int KS>
constexpr bool fits() {
    return Geo<D, KS>::LDS_BYTES <= 160 * 1024;
}
// Workgroups per CU of the kernels that keep ONE halo in LDS at a time: two where that halo
// fits twice, one for the largest halos (head_dim 128 with kernel_size 11 and 13: 88 and
// 109 KB), where these kernels are the only matrix-core ones that fit at all.
template <int D, int KS>
constexpr int kOneHaloWgs = 2 * (Geo<D, KS>::ROWS * Geo<D, KS>::PITCH * 2 + 1024) <= 160 * 1024 ? 2 : 1;
template <int D, int KS>
constexpr bool kOneHaloFits = Geo<D, KS>::ROWS * Geo<D, KS>::PITCH * 2 + 1024 <= 160 * 1024;

// ------------------------------------------------------------------ forward, one halo in LDS at a time
// The forward for halos of which LDS holds two only once per CU (head_dim 128 with
// kernel_size 7 and 9) or not at all (kernel_size 11 and 13), like bwd_dq2_mfma: K rows first
// (logits, softmax; P stays in registers as 16-bit values) while the tile's V rows are in
// flight, V over K behind a barrier, then O^T = V^T P^T while the next tile's K rows are in
// flight.  Two workgroups per CU (one at kernel_size 11 and 13), four barriers per tile; 8x8
// tiles, no column walk.
// FULL: as in fwd_mfma.
template <bool BF, int D, int KS, int NW = 4, bool FULL = false>
__global__ __launch_bounds__((Geo<D, KS, NW>::NT), (NW == 4 ? kOneHaloWgs<D, KS> : 1)) void fwd2_mfma(FwdArgs a, int tiles_r, int tiles_c, int ntiles) {
    using G = Geo<D, KS, NW>;
    __shared__ __attribute__((aligned(16))) short lds_x[G::ROWS * G::PITCH];
    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS, NW>(lds_x, dlim);

    const int wave = FULL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const HaloPlan<D, KS, NW> plan = make_plan<D, KS, NW>(dlim);
    HaloRegs<D, KS, NW> st;
    s16x8 qnext[G::DS];
    auto fetch_rows = [&](const View &vw, const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        halo_fetch<D, KS>(st, plan, image<short>(vw, tl), vw.sh, vw.sw, lq.hr0, lq.hc0, s.H, s.W);
    };
    auto fetch_q = [&](const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        load_row_chunks(qnext, image<short>(a.q, tl) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, dlim);
    };
    Tile cur = tile_of(sc.t, tiles_r, tiles_c, s.N, G::TH);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    fetch_rows(a.k, cur, lq);
    fetch_q(cur, lq);
    s16x8 qreg[G::DS];
    // (K rows and the query row at the end of a tile's pass through the loop, after its stores:
    // see fwd_mfma)
    auto commit_k = [&]() __attribute__((always_inline)) {
        halo_commit<D, KS>(lds_x, plan, st);
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) qreg[ds] = qnext[ds];
    };
    if constexpr (FULL) commit_k();
    for (;;) {
        if constexpr (!FULL) commit_k();
        __syncthreads();
        fetch_rows(a.v, cur, lq);
        auto trow = [&](int tile, int x) __attribute__((always_inline)) { return G::token_row(tile, x, lq.orow, lq.ocol); };
        s16x8 pb[G::KSTEPS];
        float mx = -INFINITY, sum = 0.f;
        if (FULL || lq.wave_on) {
            f32x4 acc[G::MT];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const typename G::ARow kp = G::a_row(lds_x, trow(mt, n), g);
                f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++)
                    c = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(kp, ds)), qreg[ds], c);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, lq.dr, lq.dc);
                    c[i] = ok ? c[i] * sc2 : -INFINITY;
                    mx = fmaxf(mx, c[i]);
                }
                acc[mt] = c;
            }
            mx = col_max(mx);
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float p = __builtin_amdgcn_exp2f(acc[mt][i] - mx);
                    sum += p;
                    pb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                }
            sum = col_sum(sum);
        }
        __syncthreads();                      // every wave has read K
        halo_commit<D, KS>(lds_x, plan, st);  // V
        __syncthreads();

        const int tn = sched_peek(sc);
        const bool more = tn < sc.t_end;
        Tile nxt = cur;
        LaneQ lqn = lq;
        if (more) {
            nxt = tile_of(tn, tiles_r, tiles_c, s.N, G::TH);
            lqn = lane_query<KS>(nxt, s, wave, n);
            fetch_rows(a.k, nxt, lqn);
            fetch_q(nxt, lqn);
        } else {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last tile, nothing is loaded (see fwd_mfma)
        }
        if (FULL || lq.wave_on) {
            f32x4 o[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) o[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                typename G::TRow vp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    vp[h] = G::t_row(lds_x, trow(ks * 2 + h, g * 4 + (n >> 2)), n);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    o[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(vp[0], mt)), lds_read_tr(G::t_at(vp[1], mt))), pb[ks],
                        o[mt]);
            }
            store_token<BF, D, kLineStores<D, KS, (NW == 4 ? kOneHaloWgs<D, KS> : 1)>, FULL>(const_cast<short *>(image<short>(a.o, cur)) + lq.qr * a.o.sh + lq.qc * a.o.sw,
                               g, o, 1.f / sum, lq.live, dlim);
            if (a.lse && (FULL || (lq.live && g == 0)))
                a.lse[lq.tok] = (mx + __builtin_amdgcn_logf(sum)) * kLn2;
        }
        if (!more) {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), see fwd_mfma
            break;
        }
        __syncthreads();  // every wave has read V
        if constexpr (FULL) commit_k();
        cur = nxt;
        lq = lqn;
        sched_advance(sc, tn);
    }
}

// ------------------------------------------------------------------ dQ
// Query-centric like the forward: recompute P from the saved log-sum-exp, form
// dP^T = V dO^T on the same halo, dS = P * (dP - delta) with delta = sum_j P_j dP_j
// (equal to dO . O, so the forward output is never read), and dQ^T = K^T dS^T with
// K read back from LDS transposed.  Also writes delta for the dK/dV pass.
// Per-query math: e_natten/triton.py:383-398.
// FRAME: walk only the tiles of the frame of `ts` (the inner tiles are served by
// the fused backward).
// head_dim 32 with kernel_size 7 and 9: the dQ pass fits the 168 registers of three waves
// per SIMD (LDS admits three workgroups per CU and more); B8 N2 112x112 k = 7: 27.8 -> 24.4
// us, B4 N4 128x128 k = 9: 37.1 -> 35.0.  The forward is as fast or faster compiled for two
// (it then takes about 150 registers and runs three per SIMD anyway).
template <int D, int KS, int NW>
constexpr int kDqWaves = D == 32 && (KS == 7 || KS == 9) && NW == 4 ? 3 : Geo<D, KS, NW>::WAVES;
// FULL: as in fwd_mfma (no wave switched off, no store predicated, the staged rows go to LDS at
// the end of a tile's pass through the loop).
template <bool BF, int D, int KS, bool FRAME, bool ROLL, int NW = 4, bool FULL = false>
__global__ __launch_bounds__((Geo<D, KS, NW>::NT), (kDqWaves<D, KS, NW>)) void bwd_dq_mfma(BwdArgs a, TileSet ts, int ntiles, Runs rp) {
    // (the dK/dV pass that follows on the stream counts its frame tiles here, from zero)
    if (blockIdx.x == 0 && threadIdx.x == 0 && a.zinv) *reinterpret_cast<int *>(a.zinv) = 0;
    using G = Geo<D, KS, NW>;
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];

    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    static_assert(!(FRAME && ROLL), "the frame is not walked by columns");
    Sched sc = ROLL ? make_runs(ntiles, blockIdx.x, gridDim.x, rp) : make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS, NW>(lds_k, dlim);
    zero_row<D, KS, NW>(lds_v, dlim);

    const int wave = FULL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    auto pick = [&](int t) __attribute__((always_inline)) {
        if constexpr (FRAME) return frame_tile(t, ts, s.N);
        else if constexpr (ROLL) return tile_of_cm(t, ts.tiles_r, ts.tiles_c, s.N);
        else return tile_of(t, ts.tiles_r, ts.tiles_c, s.N, G::TH);
    };

    const HaloPlan<D, KS, NW> plan = make_plan<D, KS, NW>(dlim);
    HaloRegs<D, KS, NW> kst, vst;
    s16x8 qnext[G::DS], gnext[G::DS];
    float lse_next = 0.f;
    // rows [y0, y0 + nr) of the halo are what LDS does not hold yet
    auto prefetch = [&](const Tile &tl, const LaneQ &lq, int y0, int nr) __attribute__((always_inline)) {
        if constexpr (ROLL) {
            halo_fetch_rows<D, KS>(kst, plan, image<short>(a.k, tl), a.k.sh, a.k.sw, y0, lq.hc0, nr, s.H, s.W);
            halo_fetch_rows<D, KS>(vst, plan, image<short>(a.v, tl), a.v.sh, a.v.sw, y0, lq.hc0, nr, s.H, s.W);
        } else {
            halo_fetch<D, KS>(kst, plan, image<short>(a.k, tl), a.k.sh, a.k.sw, lq.hr0, lq.hc0, s.H, s.W);
            halo_fetch<D, KS>(vst, plan, image<short>(a.v, tl), a.v.sh, a.v.sw, lq.hr0, lq.hc0, s.H, s.W);
        }
        load_row_chunks(qnext, image<short>(a.q, tl) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, dlim);
        load_row_chunks(gnext, image<short>(a.d_o, tl) + lq.qr * a.d_o.sh + lq.qc * a.d_o.sw, g, dlim);
        lse_next = a.lse[lq.tok];
    };

    Tile cur = pick(sc.t);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    int y0 = lq.hr0, nr = G::HR;
    prefetch(cur, lq, y0, nr);
    s16x8 qreg[G::DS], greg[G::DS];
    float lse2;
    // (at the end of a tile's pass through the loop, after its stores: see fwd_mfma)
    auto commit = [&]() __attribute__((always_inline)) {
        if constexpr (ROLL) {
            halo_commit_rows<D, KS>(lds_k, plan, kst, y0, nr);
            halo_commit_rows<D, KS>(lds_v, plan, vst, y0, nr);
        } else {
            halo_commit<D, KS>(lds_k, plan, kst);
            halo_commit<D, KS>(lds_v, plan, vst);
        }
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) {
            qreg[ds] = qnext[ds];
            greg[ds] = gnext[ds];
        }
        lse2 = lse_next * kLog2e;
    };
    if constexpr (FULL) commit();
    for (;;) {
        if constexpr (!FULL) commit();
        __syncthreads();

        const int tn = sched_peek(sc);
        const bool more = tn < sc.t_end;
        Tile nxt = cur;
        LaneQ lqn = lq;
        if (more) {
            nxt = pick(tn);
            lqn = lane_query<KS>(nxt, s, wave, n);
            // the tile below in the same image keeps the rows the two halos share
            const bool below = ROLL && nxt.bb == cur.bb && nxt.nn == cur.nn && nxt.c0 == cur.c0 &&
                               nxt.r0 > cur.r0 && lqn.hr0 < lq.hr0 + G::HR;
            y0 = below ? lq.hr0 + G::HR : lqn.hr0;
            nr = below ? lqn.hr0 - lq.hr0 : G::HR;
            prefetch(nxt, lqn, y0, nr);
        } else {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last tile, nothing is loaded (see fwd_mfma)
        }
        const int rot = ROLL ? lq.hr0 % G::HR : 0;
        auto trow = [&](int tile, int x) __attribute__((always_inline)) {
            return ROLL ? G::token_row_rot(tile, x, lq.orow, lq.ocol, rot) : G::token_row(tile, x, lq.orow, lq.ocol);
        };

        if (FULL || lq.wave_on) {
            // P^T and dP^T on the halo; delta = sum_j P_j dP_j (= dO . O) comes from
            // the same values that form dS, so sum_j dS_j vanishes to rounding
            // P is kept rounded to 16 bits (it is about to be rounded into dS
            // anyway) in the registers that will hold dS.  dP stays float32; with
            // the largest halos it is not kept but formed a second time once delta
            // is known (measured faster there: the matrix cores are idle, the
            // registers are not).
            constexpr bool kKeepDp = !(G::WAVES == 1 && G::MT >= 16);
            f32x4 dp[kKeepDp ? G::MT : 1];
            s16x8 dsb[G::KSTEPS];
            float dpart = 0.f;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const int row = trow(mt, n);
                const typename G::ARow kp = G::a_row(lds_k, row, g), vp = G::a_row(lds_v, row, g);
                f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(kp, ds)), qreg[ds], cs);
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(vp, ds)), greg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, lq.dr, lq.dc);
                    cs[i] = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - lse2 : -INFINITY);
                    dpart = fmaf(cs[i], cp[i], dpart);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(cs[i]);
                }
                if constexpr (kKeepDp) dp[mt] = cp;
            }
            const float delta = col_sum(dpart);
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                f32x4 cp;
                if constexpr (kKeepDp) {
                    cp = dp[mt];
                } else {
                    const typename G::ARow vp = G::a_row(lds_v, trow(mt, n), g);
                    cp = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ds = 0; ds < G::DS; ds++)
                        cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(vp, ds)), greg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float p = cvt32<BF>(dsb[mt >> 1][(mt & 1) * 4 + i]);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - delta));
                }
            }

            f32x4 dq[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                typename G::TRow kp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    kp[h] = G::t_row(lds_k, trow(ks * 2 + h, g * 4 + (n >> 2)), n);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    dq[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(kp[0], mt)), lds_read_tr(G::t_at(kp[1], mt))), dsb[ks],
                        dq[mt]);
            }

            store_token<BF, D, kLineStores<D, KS, G::WAVES>, FULL>(static_cast<short *>(a.dq) + a.grad_at(cur.bb, cur.nn, lq.qr, lq.qc), g, dq, s.scale, lq.live, dlim);
            if (FULL || (lq.live && g == 0)) a.delta[lq.tok] = delta;
        }

        if (!more) {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), see fwd_mfma
            break;
        }
        __syncthreads();
        if constexpr (FULL) commit();
        cur = nxt;
        lq = lqn;
        sched_advance(sc, tn);
    }
}

// ------------------------------------------------------------------ dQ, one halo in LDS at a time
// The dQ pass for halos of which LDS holds two only once per CU (head_dim 64 with
// kernel_size 13): a tile is done in two phases over ONE LDS
// buffer, so that two workgroups share a CU and each SIMD has two independent waves.
//   phase 1  V rows in LDS: dP^T = V dO^T for the wave's whole halo, kept in registers;
//            the tile's K rows are in flight meanwhile and replace V behind a barrier;
//   phase 2  K rows in LDS: P from the saved log-sum-exp, delta, dS, dQ^T = K^T dS^T;
//            the next tile's V rows are in flight meanwhile.
// Four barriers per tile instead of two; 8x8 tiles, no column walk.
// Chunks of a halo that bwd_dq2_mfma loads behind the arithmetic of a phase (see fetch_tail in
// the kernel).  With 16x8 tiles at head_dim 128, kernel_size 13 a thread stages 18 chunks (72
// registers) and the kernel spilled 70 registers, freshly loaded chunks among them, each spill
// behind a wait for its load: B4 N4 128x128 167 us; with 8 chunks behind the arithmetic 125 us,
// with 12 115.5, with 15 113.4 (5 registers spilled).  kernel_size 11: 16 chunks, 36 registers
// spilled; with 8 chunks behind the arithmetic 110.6 us, with 13 107.5.
template <int D, int KS, int NW>
constexpr int kDq2Tail = D == 128 && NW == 8 ? (KS == 13 ? 15 : KS == 11 ? 13 : 0) : 0;
// FULL: as in fwd_mfma.
template <bool BF, int D, int KS, int NW = 4, bool FULL = false>
__global__ __launch_bounds__((Geo<D, KS, NW>::NT), (NW == 4 ? kOneHaloWgs<D, KS> : 1)) void bwd_dq2_mfma(BwdArgs a, TileSet ts, int ntiles) {
    // (the dK/dV pass that follows on the stream counts its frame tiles here, from zero)
    if (blockIdx.x == 0 && threadIdx.x == 0 && a.zinv) *reinterpret_cast<int *>(a.zinv) = 0;
    using G = Geo<D, KS, NW>;
    __shared__ __attribute__((aligned(16))) short lds_x[G::ROWS * G::PITCH];
    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS, NW>(lds_x, dlim);  // (a commit only writes the halo's own rows)

    const int wave = FULL ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : threadIdx.x >> 6;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const HaloPlan<D, KS, NW> plan = make_plan<D, KS, NW>(dlim);
    HaloRegs<D, KS, NW> st;
    // This lane's dO row is loaded a phase ahead of phase 1, its q row and log-sum-exp a
    // phase ahead of phase 2: one spare set of row registers instead of two.
    s16x8 qreg[G::DS], gnext[G::DS];
    float lse_cur = 0.f;
    // The last TAIL chunks of a halo are loaded when the arithmetic of the phase is over
    // (fetch_tail): where the registers do not hold a whole halo beside it.
    constexpr int TAIL = kDq2Tail<D, KS, NW>, HEAD = G::NL - TAIL;
    auto fetch_rows = [&](const View &vw, const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        halo_fetch<D, KS, NW, 1, 0, HEAD>(st, plan, image<short>(vw, tl), vw.sh, vw.sw, lq.hr0, lq.hc0, s.H, s.W);
    };
    auto fetch_tail = [&](const View &vw, const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        if constexpr (TAIL > 0)
            halo_fetch<D, KS, NW, 1, HEAD, G::NL>(st, plan, image<short>(vw, tl), vw.sh, vw.sw, lq.hr0, lq.hc0, s.H, s.W);
    };
    auto fetch_do = [&](const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        load_row_chunks(gnext, image<short>(a.d_o, tl) + lq.qr * a.d_o.sh + lq.qc * a.d_o.sw, g, dlim);
    };
    auto fetch_q = [&](const Tile &tl, const LaneQ &lq) __attribute__((always_inline)) {
        load_row_chunks(qreg, image<short>(a.q, tl) + lq.qr * a.q.sh + lq.qc * a.q.sw, g, dlim);
        lse_cur = a.lse[lq.tok];
    };

    Tile cur = tile_of(sc.t, ts.tiles_r, ts.tiles_c, s.N, G::TH);
    LaneQ lq = lane_query<KS>(cur, s, wave, n);
    fetch_rows(a.v, cur, lq);
    fetch_tail(a.v, cur, lq);
    fetch_do(cur, lq);
    s16x8 greg[G::DS];
    // (V rows and the dO row at the end of a tile's pass through the loop, after its stores:
    // see fwd_mfma)
    auto commit_v = [&]() __attribute__((always_inline)) {
        halo_commit<D, KS>(lds_x, plan, st);
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) greg[ds] = gnext[ds];
    };
    if constexpr (FULL) commit_v();
    for (;;) {
        if constexpr (!FULL) commit_v();
        __syncthreads();
        fetch_rows(a.k, cur, lq);
        fetch_q(cur, lq);
        auto trow = [&](int tile, int x) __attribute__((always_inline)) { return G::token_row(tile, x, lq.orow, lq.ocol); };

        f32x4 dp[G::MT];
        if (FULL || lq.wave_on) {
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const typename G::ARow vp = G::a_row(lds_x, trow(mt, n), g);
                f32x4 cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++)
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(vp, ds)), greg[ds], cp);
                dp[mt] = cp;
            }
        }
        fetch_tail(a.k, cur, lq);
        __syncthreads();                      // every wave has read V
        halo_commit<D, KS>(lds_x, plan, st);  // K
        __syncthreads();

        const int tn = sched_peek(sc);
        const bool more = tn < sc.t_end;
        Tile nxt = cur;
        LaneQ lqn = lq;
        if (more) {
            nxt = tile_of(tn, ts.tiles_r, ts.tiles_c, s.N, G::TH);
            lqn = lane_query<KS>(nxt, s, wave, n);
            fetch_rows(a.v, nxt, lqn);
            fetch_do(nxt, lqn);
        } else {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the last tile, nothing is loaded (see fwd_mfma)
        }
        const float lse2 = lse_cur * kLog2e;
        if (FULL || lq.wave_on) {
            s16x8 dsb[G::KSTEPS];
            float dpart = 0.f;
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                const typename G::ARow kp = G::a_row(lds_x, trow(mt, n), g);
                f32x4 cs = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++)
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(kp, ds)), qreg[ds], cs);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, lq.dr, lq.dc);
                    const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - lse2 : -INFINITY);
                    dpart = fmaf(p, dp[mt][i], dpart);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                }
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
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                typename G::TRow kp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    kp[h] = G::t_row(lds_x, trow(ks * 2 + h, g * 4 + (n >> 2)), n);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    dq[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(kp[0], mt)), lds_read_tr(G::t_at(kp[1], mt))), dsb[ks],
                        dq[mt]);
            }
            store_token<BF, D, kLineStores<D, KS, (NW == 4 ? kOneHaloWgs<D, KS> : 1)>, FULL>(static_cast<short *>(a.dq) + a.grad_at(cur.bb, cur.nn, lq.qr, lq.qc), g, dq, s.scale, lq.live, dlim);
            if (FULL || (lq.live && g == 0)) a.delta[lq.tok] = delta;
        }
        if (more) fetch_tail(a.v, nxt, lqn);
        if (!more) {
            if constexpr (FULL) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0), see fwd_mfma
            break;
        }
        __syncthreads();  // every wave has read K
        if constexpr (FULL) commit_v();
        cur = nxt;
        lq = lqn;
        sched_advance(sc, tn);
    }
}

// ------------------------------------------------------------------ dK, dV
// Key-centric: the workgroup owns an 8x8 tile of keys and stages Q, dO, the
// log-sum-exp and delta of the queries that attend to them, i.e. the union of the
// keys' inverse neighbourhoods (e_natten/pytorch.py:13-23, :261-270).  That union
// is (8+k-1)^2 queries in the interior and larger beside an image edge (the
// clamped windows of the k//2 border queries all reach k pixels in), so it is
// walked in blocks of at most (8+k-1)^2 queries; a block is the unit that is
// staged in LDS and prefetched.  Each wave owns 4x4 keys (MFMA columns) and walks
// the queries of the block that can attend to them, 32 at a time:
//   S = Q K^T, dP = dO V^T           (query rows from LDS, key columns in registers)
//   P = exp(S - lse), dS = P (dP - delta), masked to the query's own window
//   dV^T += dO^T P, dK^T += Q^T dS    (dO, Q read back from LDS transposed)
struct KeyBlock {
    int t;                // tile
    Tile tl;
    int qa, qb, ca, cb;   // queries that attend to any key of the tile
    int br, bc;           // origin of the staged block of queries
    bool first, last;     // first / last block of its tile
};
// Next block of the same tile, or false when the tile is finished.
template <int HR, int HC>
__device__ __forceinline__ bool next_block(KeyBlock &b) {
    if (b.last) return false;
    b.first = false;
    b.bc += HC;
    if (b.bc >= b.cb) {
        b.bc = b.ca;
        b.br += HR;
    }
    b.last = b.br + HR >= b.qb && b.bc + HC >= b.cb;
    return true;
}


// Inner tiles.  Every key is attended by exactly the queries within k//2 of it
// and all windows are centred, so the picture is the forward's with the roles of
// queries and keys exchanged: the staged block is the tile's (8+k-1)^2 halo of
// queries, a wave's queries are the (4+k-1)^2 halo of its 4x4 keys at a fixed
// place in it, and the mask depends on the lane only.
template <bool BF, int D, int KS, bool ROLL, int SP, int PART>
__device__ __forceinline__ void dkdv_inner(const BwdArgs &a, const TileSet &ts, int ntiles, Runs rp,
                                           int block, int nblocks, short *lds_q, short *lds_g,
                                           float2 *lds_stat, f32x4 *lds_red) {
    using G = Geo<D, KS, 4, SP>;
    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    Sched sc = ROLL ? make_runs(ntiles, block, nblocks, rp) : make_sched(ntiles, block, nblocks);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS, 4, SP>(lds_q, dlim);
    zero_row<D, KS, 4, SP>(lds_g, dlim);
    if (threadIdx.x == 0) lds_stat[G::ZROW] = make_float2(0.f, 0.f);

    // wave = block of 4x4 keys (0..3) + 4 * PART; part p takes reduction steps
    // K0 = p * CH .. K1 - 1 (compile-time, so that every token's place in the halo and its
    // mask fold to constants)
    const int wave = SP == 1 ? threadIdx.x >> 6 : (threadIdx.x >> 6) & 3;
    constexpr int part = PART;
    constexpr int CH = (G::KSTEPS + SP - 1) / SP;
    constexpr int K0 = PART * CH, K1 = K0 + CH < G::KSTEPS ? K0 + CH : G::KSTEPS;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;
    const int orow = (wave >> 1) * 4, ocol = (wave & 1) * 4;
    int rot = 0;  // ROLL: (first image row of the staged block) % HR
    auto row_of = [&](int tile, int x) __attribute__((always_inline)) {
        return ROLL ? G::token_row_rot(tile, x, orow, ocol, rot) : G::token_row(tile, x, orow, ocol);
    };
    auto pick = [&](int t) __attribute__((always_inline)) {
        return ROLL ? inner_tile_cm(t, ts, s.N) : inner_tile(t, ts, s.N);
    };

    const HaloPlan<D, KS, 4, SP> plan = make_plan<D, KS, 4, SP>(dlim);
    HaloRegs<D, KS, 4, SP> qst, gst;
    float2 sst[G::NST];
    // ROLL: rows [y0, y0 + nr) of the block are what LDS does not hold yet
    auto prefetch = [&](const Tile &tl, int y0, int nr) __attribute__((always_inline)) {
        const int64_t img_tok = ((int64_t)tl.bb * s.N + tl.nn) * s.H * (int64_t)s.W;
        const int br = tl.r0 - KS / 2, bc = tl.c0 - KS / 2;
        if constexpr (ROLL) {
            halo_fetch_rows<D, KS>(qst, plan, image<short>(a.q, tl), a.q.sh, a.q.sw, y0, bc, nr, s.H, s.W);
            halo_fetch_rows<D, KS>(gst, plan, image<short>(a.d_o, tl), a.d_o.sh, a.d_o.sw, y0, bc, nr, s.H, s.W);
        } else {
            halo_fetch<D, KS>(qst, plan, image<short>(a.q, tl), a.q.sh, a.q.sw, br, bc, s.H, s.W);
            halo_fetch<D, KS>(gst, plan, image<short>(a.d_o, tl), a.d_o.sh, a.d_o.sw, br, bc, s.H, s.W);
        }
#pragma unroll
        for (int i = 0; i < G::NST; i++) {
            const int id = min((int)threadIdx.x + i * G::NT, G::ZROW - 1);
            const int pr = id / G::HC, pc = id % G::HC;
            if (!ROLL || pr < nr) {
                const int64_t qt = img_tok + (int64_t)((ROLL ? y0 : br) + pr) * s.W + bc + pc;
                sst[i] = make_float2(a.lse[qt] * kLog2e, a.delta[qt]);
            }
        }
    };
    auto commit = [&](int y0, int nr) __attribute__((always_inline)) {
        if constexpr (ROLL) {
            halo_commit_rows<D, KS>(lds_q, plan, qst, y0, nr);
            halo_commit_rows<D, KS>(lds_g, plan, gst, y0, nr);
            const int r0m = y0 % G::HR;
#pragma unroll
            for (int i = 0; i < G::NST; i++) {
                const int id = threadIdx.x + i * G::NT;
                const int pr = id / G::HC, pc = id % G::HC;
                if (id < G::ZROW && pr < nr) {
                    int slot = r0m + pr;
                    slot = slot >= G::HR ? slot - G::HR : slot;
                    lds_stat[slot * G::HC + pc] = sst[i];
                }
            }
        } else {
            halo_commit<D, KS>(lds_q, plan, qst);
            halo_commit<D, KS>(lds_g, plan, gst);
#pragma unroll
            for (int i = 0; i < G::NST; i++) {
                const int id = threadIdx.x + i * G::NT;
                if (id < G::ZROW) lds_stat[id] = sst[i];
            }
        }
    };
    // B operands of a tile: this lane's key, channels ds*32 + g*8 ..  Loaded when
    // the previous tile's math is over (they would not fit beside it) and complete
    // before the barrier below, i.e. before any newer load is in flight.
    s16x8 kreg[G::DS], vreg[G::DS];
    auto load_keys = [&](const Tile &tl) __attribute__((always_inline)) {
        const int kr = tl.r0 + orow + (n >> 2), kc = tl.c0 + ocol + (n & 3);
        load_row_chunks(kreg, image<short>(a.k, tl) + kr * a.k.sh + kc * a.k.sw, g, dlim);
        load_row_chunks(vreg, image<short>(a.v, tl) + kr * a.v.sh + kc * a.v.sw, g, dlim);
    };

    Tile cur = pick(sc.t);
    int y0 = cur.r0 - KS / 2, nr = G::HR;
    prefetch(cur, y0, nr);
    load_keys(cur);
    for (;;) {
        commit(y0, nr);
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) asm volatile("" : "+v"(kreg[ds]), "+v"(vreg[ds]));
        __syncthreads();

        const int tn = sched_peek(sc);
        const bool more = tn < sc.t_end;
        Tile nxt = cur;
        if (ROLL) rot = (cur.r0 - KS / 2) % G::HR;
        if (more) {
            nxt = pick(tn);
            // the tile below in the same image keeps the rows the two blocks share
            const bool below = ROLL && nxt.bb == cur.bb && nxt.nn == cur.nn && nxt.c0 == cur.c0 &&
                               nxt.r0 > cur.r0 && nxt.r0 - cur.r0 < G::HR;
            y0 = below ? cur.r0 - KS / 2 + G::HR : nxt.r0 - KS / 2;
            nr = below ? nxt.r0 - cur.r0 : G::HR;
            prefetch(nxt, y0, nr);
        }

        f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
        for (int mt = 0; mt < G::DT; mt++) {
            dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int ks = K0; ks < K1; ks++) {
            s16x8 pb, dsb;
#pragma unroll
            for (int m2 = 0; m2 < 2; m2++) {
                const int mt = ks * 2 + m2;
                const int row = row_of(mt, n);
                const typename G::ARow qp = G::a_row(lds_q, row, g), gp = G::a_row(lds_g, row, g);
                f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(qp, ds)), kreg[ds], cs);
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(gp, ds)), vreg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float2 st = lds_stat[row_of(mt, g * 4 + i)];  // query of accumulator row g*4+i
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, n >> 2, n & 3);
                    const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
                    pb[m2 * 4 + i] = cvt16<BF>(p);
                    dsb[m2 * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                }
            }
            typename G::TRow qt[2], gt[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int row = row_of(ks * 2 + h, g * 4 + (n >> 2));
                qt[h] = G::t_row(lds_q, row, n);
                gt[h] = G::t_row(lds_g, row, n);
            }
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) {
                dv[mt] = mfma16<BF>(cat(lds_read_tr(G::t_at(gt[0], mt)), lds_read_tr(G::t_at(gt[1], mt))),
                                    pb, dv[mt]);
                dk[mt] = mfma16<BF>(cat(lds_read_tr(G::t_at(qt[0], mt)), lds_read_tr(G::t_at(qt[1], mt))),
                                    dsb, dk[mt]);
            }
        }

        const int kr = cur.r0 + orow + (n >> 2), kc = cur.c0 + ocol + (n & 3);
        const int64_t goff = a.grad_at(cur.bb, cur.nn, kr, kc);
        if constexpr (SP == 1) {
            store_token<BF, D, kInnerLines<D>, true>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, true, dlim);
            store_token<BF, D, kInnerLines<D>, true>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, true, dlim);
            if (!more) break;
            load_keys(nxt);
            __syncthreads();
        } else {
            // the second part hands its sums to the first through LDS; the first adds
            // and stores them once the barrier that ends the tile has passed (the
            // second part writes again only after the next tile's first barrier)
            static_assert(SP <= 2, "two parts");
            f32x4 *red = lds_red + wave * 64 + l;
            if (part == 1) {
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    red[mt * 256] = dk[mt];
                    red[(G::DT + mt) * 256] = dv[mt];
                }
            }
            if (more) load_keys(nxt);
            __syncthreads();
            if (part == 0) {
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dk[mt] += red[mt * 256];
                    dv[mt] += red[(G::DT + mt) * 256];
                }
                store_token<BF, D, kInnerLines<D>, true>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, true, dlim);
                store_token<BF, D, kInnerLines<D>, true>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, true, dlim);
            }
            if (!more) break;
        }
        cur = nxt;
        sched_advance(sc, tn);
    }
}

// Frame tiles: the general case, walked block by block (see above).  KSG sets the size of a
// staged block, (8 + KSG - 1)^2 queries: KS, or more (kFrameKS) so that the queries of a
// tile in the second ring from the border, up to 16 + k/2 rows and columns of them, are
// one block instead of up to four.  `lds_red` then lies over the staged rows (RED_OVER):
// the partial sums are exchanged when a tile's last block has been read by every wave.
template <bool BF, int D, int KS, int SP, int KSG, bool RED_OVER>
__device__ __forceinline__ void dkdv_frame(const BwdArgs &a, const TileSet &ts, int ntiles,
                                           int block, int nblocks, short *lds_q, short *lds_g,
                                           float4 *lds_stat, f32x4 *lds_red, int *tile_ctr, int *lds_tile) {
    using G = Geo<D, KSG, 4, SP>;
    const Shape &s = a.s;
    const int dlim = kNarrow ? s.D : D;  // head dim of the tensors: D, or less in the build for narrow dims
    // Tiles: a strided share of the XCD's run (make_sched), or, with a counter in device memory
    // that is zero when the kernel starts (`tile_ctr`), whatever tile is next when the workgroup
    // is free.  A workgroup then knows its tile and the one after it, and asks for the tile after
    // those while it works on a tile's first block, so the answer never holds it up.
    const bool dyn = tile_ctr != nullptr;
    Sched sc = make_sched(ntiles, block, nblocks);
    int t_next = sc.t + sc.step;
    if (dyn) {
        if (threadIdx.x == 0) {
            lds_tile[0] = atomicAdd(tile_ctr, 1);
            lds_tile[1] = atomicAdd(tile_ctr, 1);
        }
        __syncthreads();
        sc.t = lds_tile[0];
        t_next = lds_tile[1];
        sc.t_end = ntiles;
    }
    if (sc.t >= sc.t_end) return;
    zero_row<D, KSG, 4, SP>(lds_q, dlim);
    zero_row<D, KSG, 4, SP>(lds_g, dlim);

    // wave = block of 4x4 keys (0..3) + 4 * (its part of the block's queries)
    const int wave = (threadIdx.x >> 6) & 3, part = threadIdx.x >> 8;
    const int l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const float sc2 = s.scale * kLog2e;

    const HaloPlan<D, KSG, 4, SP> plan = make_plan<D, KSG, 4, SP>(dlim);
    HaloRegs<D, KSG, 4, SP> qst, gst;
    float2 sst[G::NST];
    // the wave's 4x4 keys of a tile: this lane's key pixel (clamped into the image)
    auto key_of = [&](const Tile &tl, int &kr, int &kc) __attribute__((always_inline)) {
        kr = min(tl.r0 + (wave >> 1) * 4 + (n >> 2), s.H - 1);
        kc = min(tl.c0 + (wave & 1) * 4 + (n & 3), s.W - 1);
    };
    auto stage = [&](const KeyBlock &b) __attribute__((always_inline)) {
        const int64_t img_tok = ((int64_t)b.tl.bb * s.N + b.tl.nn) * s.H * (int64_t)s.W;
        halo_fetch<D, KSG>(qst, plan, image<short>(a.q, b.tl), a.q.sh, a.q.sw, b.br, b.bc, b.qb, b.cb);
        halo_fetch<D, KSG>(gst, plan, image<short>(a.d_o, b.tl), a.d_o.sh, a.d_o.sw, b.br, b.bc, b.qb, b.cb);
#pragma unroll
        for (int i = 0; i < G::NST; i++) {
            const int id = threadIdx.x + i * G::NT;
            const int r = min(b.br + id / G::HC, b.qb - 1), c = min(b.bc + id % G::HC, b.cb - 1);
            const int64_t qt = img_tok + (int64_t)r * s.W + c;
            sst[i] = make_float2(a.lse[qt] * kLog2e, a.delta[qt]);
        }
    };
    // B operands of the tile: this lane's key, channels ds*32 + g*8 ..
    s16x8 kreg[G::DS], vreg[G::DS];
    auto load_keys = [&](const Tile &tl) __attribute__((always_inline)) {
        int kr, kc;
        key_of(tl, kr, kc);
        load_row_chunks(kreg, image<short>(a.k, tl) + kr * a.k.sh + kc * a.k.sw, g, dlim);
        load_row_chunks(vreg, image<short>(a.v, tl) + kr * a.v.sh + kc * a.v.sw, g, dlim);
    };
    auto first_of = [&](int t) __attribute__((always_inline)) {
        KeyBlock b;
        b.t = t;
        b.tl = frame_tile(t, ts, s.N);
        b.qa = inv_lo(b.tl.r0, KS);
        b.qb = inv_hi(min(b.tl.r0 + 8, s.H) - 1, s.H, KS);
        b.ca = inv_lo(b.tl.c0, KS);
        b.cb = inv_hi(min(b.tl.c0 + 8, s.W) - 1, s.W, KS);
        b.br = b.qa;
        b.bc = b.ca;
        b.first = true;
        b.last = b.br + G::HR >= b.qb && b.bc + G::HC >= b.cb;
        return b;
    };

    f32x4 dk[G::DT], dv[G::DT];
    KeyBlock cur = first_of(sc.t);
    // With one part per block (SP == 1) the loads of a block are issued when the previous
    // block's math is over and the other workgroup on the CU covers their latency
    // (keeping them in flight across the math would need registers that the two
    // accumulators do not leave).  With two parts a thread stages half as much, and the
    // next block's loads are in flight while this one is computed.
    stage(cur);
    load_keys(cur.tl);
    for (;;) {
        int fetched = 0;
        if (dyn && cur.first && threadIdx.x == 0) fetched = atomicAdd(tile_ctr, 1);
        halo_commit<D, KSG>(lds_q, plan, qst);
        halo_commit<D, KSG>(lds_g, plan, gst);
#pragma unroll
        for (int i = 0; i < G::NST; i++) {
            const int id = threadIdx.x + i * G::NT;
            // per staged query: lse * log2e, delta, and where its window starts (row in the low,
            // column in the high half of a word), so that the mask of a logit is two
            // differences; the padding row's window is nowhere
            const int r = min(cur.br + id / G::HC, cur.qb - 1), c = min(cur.bc + id % G::HC, cur.cb - 1);
            const int ws = win_start(r, s.H, KS) | (win_start(c, s.W, KS) << 16);
            if (id < G::ZROW) lds_stat[id] = make_float4(sst[i].x, sst[i].y, __int_as_float(ws), 0.f);
            else if (id == G::ZROW) lds_stat[id] = make_float4(0.f, 0.f, __int_as_float(0x7fff7fff), 0.f);
        }
        if (cur.first) {
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) {
                dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        __syncthreads();

        KeyBlock nxt = cur;
        bool more = next_block<G::HR, G::HC>(nxt);
        if (!more && t_next < sc.t_end) {
            nxt = first_of(t_next);
            more = true;
        }
        if constexpr (SP > 1) {
            if (more) stage(nxt);
        }
        const int wr0 = cur.tl.r0 + (wave >> 1) * 4, wc0 = cur.tl.c0 + (wave & 1) * 4;
        const bool wave_on = wr0 < s.H && wc0 < s.W;
        int kr, kc;
        key_of(cur.tl, kr, kc);
        if (wave_on) {
            // this wave's queries inside the staged block: those that attend to any
            // of its 4x4 keys, numbered row-major over their rectangle
            const int ra = max(inv_lo(wr0, KS), cur.br);
            const int rb = min(inv_hi(min(wr0 + 4, s.H) - 1, s.H, KS), cur.br + G::HR);
            const int cc = max(inv_lo(wc0, KS), cur.bc);
            const int cd = min(inv_hi(min(wc0 + 4, s.W) - 1, s.W, KS), cur.bc + G::HC);
            const int wcols = cd - cc;
            const int nq = (rb > ra && cd > cc) ? (rb - ra) * wcols : 0;
            // qi * magic >> 16 == qi / wcols for qi < 2048, wcols <= 32
            const int magic = wcols > 0 ? (65536 + wcols - 1) / wcols : 0;
            // staged row of query qi (zero row past the end), branch-free
            auto row_of = [&](int qi) __attribute__((always_inline)) {
                const int dvd = (qi * magic) >> 16;
                const int row = (ra + dvd - cur.br) * G::HC + (cc + qi - dvd * wcols - cur.bc);
                return qi < nq ? row : (int)G::ZROW;
            };
            for (int q0 = part * 32; q0 < nq; q0 += 32 * SP) {
                s16x8 pb, dsb;
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++) {
                    const int row = row_of(q0 + m2 * 16 + n);
                    const typename G::ARow qp = G::a_row(lds_q, row, g), gp = G::a_row(lds_g, row, g);
                    f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ds = 0; ds < G::DS; ds++) {
                        cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(qp, ds)), kreg[ds], cs);
                        cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(gp, ds)), vreg[ds], cp);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int qi = q0 + m2 * 16 + g * 4 + i;
                        const float4 st = lds_stat[row_of(qi)];
                        const int ws = __float_as_int(st.z);
                        const bool ok = ((unsigned)(kr - (ws & 0xffff)) < (unsigned)KS) &
                                        ((unsigned)(kc - (ws >> 16)) < (unsigned)KS);
                        const float p =
                            __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
                        pb[m2 * 4 + i] = cvt16<BF>(p);
                        dsb[m2 * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                    }
                }
                typename G::TRow qt[2], gt[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int row = row_of(q0 + h * 16 + g * 4 + (n >> 2));
                    qt[h] = G::t_row(lds_q, row, n);
                    gt[h] = G::t_row(lds_g, row, n);
                }
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dv[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(gt[0], mt)), lds_read_tr(G::t_at(gt[1], mt))), pb, dv[mt]);
                    dk[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(qt[0], mt)), lds_read_tr(G::t_at(qt[1], mt))), dsb, dk[mt]);
                }
            }
        }

        // (read below, behind the barrier that ends this block; the first block of the next tile
        // writes it again behind the barrier that opens its arithmetic)
        if (dyn && cur.first && threadIdx.x == 0) lds_tile[0] = fetched;
        const bool live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
        auto store = [&]() __attribute__((always_inline)) {
            const int64_t goff = a.grad_at(cur.tl.bb, cur.tl.nn, kr, kc);
            store_token<BF, D, kLineStores<D, KS, fits<D, KS>() ? Geo<D, KS, 4, SP>::WAVES : 1>>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, live, dlim);
            store_token<BF, D, kLineStores<D, KS, fits<D, KS>() ? Geo<D, KS, 4, SP>::WAVES : 1>>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, live, dlim);
        };
        if constexpr (SP == 1) {
            if (cur.last) store();
            if (!more) break;
            stage(nxt);
            if (nxt.first) load_keys(nxt.tl);
            __syncthreads();
        } else {
            // the second part's sums reach the first through LDS (see dkdv_inner)
            f32x4 *red = lds_red + wave * 64 + l;
            if (RED_OVER && cur.last) __syncthreads();  // every wave has read the block
            if (cur.last && part == 1) {
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    red[mt * 256] = dk[mt];
                    red[(G::DT + mt) * 256] = dv[mt];
                }
            }
            if (more && nxt.first) load_keys(nxt.tl);
            __syncthreads();
            if (cur.last && part == 0) {
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dk[mt] += red[mt * 256];
                    dv[mt] += red[(G::DT + mt) * 256];
                }
                store();
            }
            if (!more) break;
            if (RED_OVER && cur.last) __syncthreads();  // the sums are read: the next block may land
        }
        if (nxt.first) t_next = dyn ? lds_tile[0] : nxt.t + sc.step;  // the tile after the next one
        cur = nxt;
    }
}

// One launch for the whole dK/dV pass: the first `inner_blocks` workgroups sweep
// the inner tiles, the rest the frame tiles, so the two kinds of work overlap on
// every CU and end together.
// SP = 2: eight waves, two per 4x4 block of keys (see Geo), for halos that leave LDS for
// one workgroup per CU.
// Waves per SIMD that the dK/dV pass budgets its registers for: three where LDS admits
// three workgroups per CU (head_dim <= 64 with small halos; it fits 168 registers there,
// measured 35 -> 32 us at B8 N2 112x112 d32 k7 and 67 -> 60 us at B4 N4 128x128 d32 k9;
// the forward and the dQ pass spill under that budget and get slower).
// Size of the frame body's blocks as a kernel size (see dkdv_frame): larger than KS where the
// pass has one workgroup per CU anyway (two parts per block) and LDS has the room.
// Where not even one workgroup's Q and dO halos fit LDS (head_dim 128 with kernel_size 11 and
// 13), the pass has no inner body: EVERY tile is walked by the frame body in blocks of 12x12
// queries (78 KB for both tensors, two workgroups per CU), four to nine blocks per tile.
template <int D, int KS>
constexpr bool kDkdvFrameOnly = !fits<D, KS>();
template <int D, int KS, int SP>
constexpr int kFrameKS = kDkdvFrameOnly<D, KS> ? 5 : SP == 2 && KS >= 9 ? 9 + KS / 2 : KS;
template <int D, int KS, int SP>
constexpr int kDkdvWaves =
    kDkdvFrameOnly<D, KS> ? 2 :
    SP == 1 && D <= 64 && 3 * (Geo<D, KS>::LDS_BYTES + 2048) <= 160 * 1024 ? 3 : Geo<D, KS, 4, SP>::WAVES;
template <bool BF, int D, int KS, bool ROLL, int SP = 1>
__global__ __launch_bounds__((Geo<D, KS, 4, SP>::NT), (kDkdvWaves<D, KS, SP>)) void bwd_dkdv_mfma(
    BwdArgs a, TileSet ts, int n_inner, int n_frame, int inner_blocks, Runs rp, int dyn) {
    using G = Geo<D, KS, 4, SP>;
    using FG = Geo<D, kFrameKS<D, KS, SP>, 4, SP>;  // blocks of the frame body
    // One LDS buffer, laid out by each body for itself: staged Q rows, staged dO rows,
    // (lse * log2e, delta) per staged query, and with two parts per block the second part's
    // partial dK and dV.  Where the frame body stages larger blocks, its partial sums lie
    // over its Q rows.
    constexpr bool FRAME_ONLY = kDkdvFrameOnly<D, KS>;
    constexpr bool RED_OVER = !std::is_same<FG, G>::value && !FRAME_ONLY;
    constexpr size_t RED = SP > 1 ? (size_t)2 * G::DT * 256 * sizeof(f32x4) : 0;
    constexpr size_t I_ROWS = FRAME_ONLY ? 0 : (size_t)G::ROWS * G::PITCH * sizeof(short);
    constexpr size_t F_ROWS = (size_t)FG::ROWS * FG::PITCH * sizeof(short);
    constexpr size_t I_STAT = FRAME_ONLY ? 0 : (G::ROWS * sizeof(float2) + 15) / 16 * 16;
    constexpr size_t F_STAT = FG::ROWS * sizeof(float4);
    constexpr size_t I_ALL = 2 * I_ROWS + I_STAT + RED;
    constexpr size_t F_ALL = 2 * F_ROWS + F_STAT + (RED_OVER ? 0 : RED);
    static_assert(RED <= F_ROWS || !RED_OVER, "the partial sums lie over the staged Q rows");
    __shared__ __attribute__((aligned(16))) char lds_raw[I_ALL > F_ALL ? I_ALL : F_ALL];
    static_assert(sizeof(lds_raw) <= 160 * 1024, "LDS");
    // dyn: the frame tiles are dealt out as workgroups become free, the inner workgroups joining
    // when their walk is over; the counter lies where the general kernels keep 1 / Z per query,
    // and the dQ pass, which runs before this one on the stream, has cleared it.
    __shared__ int lds_tile[2];
    int *tile_ctr = dyn ? reinterpret_cast<int *>(a.zinv) : nullptr;
    if constexpr (!FRAME_ONLY) {
        if ((int)blockIdx.x < inner_blocks) {
            short *lds_q = reinterpret_cast<short *>(lds_raw);
            short *lds_g = reinterpret_cast<short *>(lds_raw + I_ROWS);
            float2 *lds_stat = reinterpret_cast<float2 *>(lds_raw + 2 * I_ROWS);
            f32x4 *lds_red = reinterpret_cast<f32x4 *>(lds_raw + 2 * I_ROWS + I_STAT);
            if (SP == 1 || threadIdx.x < 256)
                dkdv_inner<BF, D, KS, ROLL, SP, 0>(a, ts, n_inner, rp, blockIdx.x, inner_blocks, lds_q,
                                                   lds_g, lds_stat, lds_red);
            else  // the same number of barriers as the first part
                dkdv_inner<BF, D, KS, ROLL, SP, SP - 1>(a, ts, n_inner, rp, blockIdx.x, inner_blocks,
                                                        lds_q, lds_g, lds_stat, lds_red);
            if (!dyn) return;
            __syncthreads();
        }
    }
    {
        short *lds_q = reinterpret_cast<short *>(lds_raw);
        short *lds_g = reinterpret_cast<short *>(lds_raw + F_ROWS);
        float4 *lds_stat = reinterpret_cast<float4 *>(lds_raw + 2 * F_ROWS);
        f32x4 *lds_red = reinterpret_cast<f32x4 *>(RED_OVER ? lds_raw : lds_raw + 2 * F_ROWS + F_STAT);
        dkdv_frame<BF, D, KS, SP, kFrameKS<D, KS, SP>, RED_OVER>(
            a, ts, n_frame, dyn ? blockIdx.x : blockIdx.x - inner_blocks,
            dyn ? gridDim.x : gridDim.x - inner_blocks, lds_q, lds_g, lds_stat, lds_red, tile_ctr, lds_tile);
    }
}

// ------------------------------------------------------------------ dispatch

// Keeping shared halo rows in LDS pays where the kernels are bound by the bytes
// they pull through the CU's memory pipeline (d = 128) and a workgroup walks at
// least a few tiles down a column; elsewhere its extra address arithmetic costs
// more than the loads it saves (measured), so it is only built for d = 128.
template <int D>
constexpr bool kRollBuilt = D == 128;
template <int D>
bool roll_pays(int64_t ntiles, int grid) {
    return kRollBuilt<D> && ntiles >= (int64_t)4 * grid;
}

// Eight waves on a 16x8 tile instead of four on an 8x8 tile, for head_dim 64 with
// kernel_size >= 7 where the taller tile's halo fits LDS: a fifth to a third less halo
// per pixel, and at k = 11 and 13, where the halo of an 8x8 tile leaves LDS for one
// workgroup per CU, two waves per SIMD instead of one.  Measured at B4 N4 128x128
// (8x8 -> 16x8, us): forward 40 -> 39 (k=7), 76 -> 53 (k=11), 82 -> 55 (k=13); dQ pass
// 59 -> 48 (k=7), 82 -> 59 (k=9).  Not used where it was measured slower or no faster:
// k <= 5, head_dim 32, and the dQ pass at k = 11 and 13, where the pass with one halo in
// LDS at a time (bwd_dq2_mfma) is faster (k = 11: 87 us against 75; at k = 13 the 16x8
// tiles spill).
template <int D, int KS>
constexpr bool kTallBuilt =
    D == 64 && KS >= 7 &&
    (size_t)2 * Geo<D, KS, 8>::ROWS * Geo<D, KS, 8>::PITCH * sizeof(short) <= 160 * 1024;
template <int D, int KS>
constexpr bool kTallDqBuilt = kTallBuilt<D, KS> && KS <= 9;

// The dQ pass with one halo in LDS at a time (bwd_dq2_mfma): where two halos leave LDS for
// one workgroup per CU, one halo fits twice, and the 16x8 tiles are not used.  head_dim 64
// (kernel_size 11 and 13): 96 -> 79 us at B2 N8 128x128 k = 13; k = 11, against the 16x8
// tiles: 87.3 -> 75.2 us at B4 N4 128x128, 380 -> 296 at 256x256, 27.0 -> 23.1 at B2 N8 64x64.  head_dim 128 (kernel_size 7 and 9), B4 N4
// 128x128: 110.6 -> 72.2 us and 123.8 -> 80.3; B8 N8: 431 -> 302; B2 N2 64x64: 10.9 -> 10.1.
template <int D, int KS>
constexpr bool kDq2Built = (D == 64 || D == 128) && Geo<D, KS>::WAVES == 1 && !kTallDqBuilt<D, KS> &&
                           kOneHaloFits<D, KS>;

// The forward with one halo in LDS at a time (fwd2_mfma), for head_dim 128 where two halos
// leave LDS for one workgroup per CU (kernel_size 7 and 9).  Launched where the tiles give
// every CU its two workgroups (us, fwd_mfma -> fwd2_mfma, bf16, 128x128 images): k = 7
// B1 N2 14.1 -> 12.5, B1 N4 26.3 -> 20.3, B4 N4 91.8 -> 60.5, B8 N8 364 -> 245; k = 9
// B1 N4 28.0 -> 22.4, B4 N4 106.6 -> 68.5.  With fewer tiles fwd_mfma's single workgroup
// per CU is faster (B2 N2 64x64: 9.3 us against 9.9).  At head_dim 64 (kernel_size 11, 13)
// the 16x8 tiles of fwd_mfma are faster (57.8 us against 59.3, 61.6 against 69.5).
// 16x8 tiles with eight waves for the one-halo kernels where an 8x8 tile's halo leaves LDS for one
// workgroup of four waves per CU (head_dim 128, kernel_size 11 and 13) and the taller halo still
// fits (128 and 153 KB): two waves per SIMD instead of one, and a quarter less halo per pixel.
// B4 N4 128x128, us, 8x8 -> 16x8: forward k13 137.8 -> 104.5 (B8 N8: 526 -> 385), k11 143.4 -> 130.4;
// dQ pass k13 179.7 -> 167.7 (B8 N8: 736 -> 642), k11 185.2 -> 190.4 while it spilled 70 and 36
// registers there; with the last chunks of a halo loaded behind the arithmetic (kDq2Tail) it
// does not, and the tall tiles take k13 to 113 us and k11 to 107.5 (174 with 8x8 tiles; B8 N8:
// 700 -> 426).
template <int D, int KS>
constexpr bool kFwd2TallBuilt = D == 128 && kOneHaloWgs<D, KS> == 1 && kOneHaloFits<D, KS> &&
                                (size_t)Geo<D, KS, 8>::ROWS * Geo<D, KS, 8>::PITCH * 2 + 1024 <= 160 * 1024;
// At head_dim 64 (kernel_size 11 and 13, where one halo of an 8x8 tile fits LDS twice) the one-halo dQ
// pass takes the 16x8 tiles too: one workgroup of eight waves instead of two of four, a quarter less halo
// per pixel.  B2 N8 128x128 k13 81.5 -> 76.2 us, B4 N8 256x256 626 -> 606, B4 N4 128x128 k11 77.1 -> 76.3.
template <int D, int KS>
constexpr bool kDq2TallBuilt = kFwd2TallBuilt<D, KS> || (D == 64 && KS >= 11);
template <int D, int KS>
constexpr bool kFwd2Built = D == 128 && Geo<D, KS>::WAVES == 1 && kOneHaloFits<D, KS>;
// Built at all: two halos fit, or the one-halo kernels serve the forward and the dQ pass and
// the frame body in small blocks the dK/dV pass
template <int D, int KS>
constexpr bool kBuilt = fits<D, KS>() || (kFwd2Built<D, KS> && kDq2Built<D, KS>);

// A frame tile's time in inner tiles in the dK/dV pass at head_dim 128, as the choice of the
// split takes it (bwd_launch).  Measured over six image sizes from 64x64 to 256x256 with the
// weights 0.8 to 4.0: 1.3 and 1.6 are within 1% of each other at k = 3, 5 and 7; at k = 9, where
// the frame is two tiles wide, 2.0 is the best or within 3% of it everywhere (B4 N4 128x128: 227 us
// with 1.15, 245 with 1.6, 176 with 2.0; B2 N2 256x256: 223, 167, 155).
template <int KS>
constexpr double kFrameCost128 = KS >= 9 ? 2.0 : KS == 5 ? 1.45 : 1.3;
template <int D, int KS>
constexpr int kDkdvSplit = D == 64 && Geo<D, KS>::WAVES == 1 ? 2 : 1;

template <bool BF, int D, int KS>
int fwd_launch(const FwdArgs &a, hipStream_t st) {
    if constexpr (kBuilt<D, KS>) {
        using G = Geo<D, KS>;
        const int tiles_r = (a.s.H + G::TH - 1) / G::TH, tiles_c = (a.s.W + G::TW - 1) / G::TW;
        const int64_t nb = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
        if constexpr (kTallBuilt<D, KS>) {
            using G8 = Geo<D, KS, 8>;
            const int tall_r = (a.s.H + G8::TH - 1) / G8::TH;
            const int64_t nb8 = (int64_t)a.s.B * a.s.N * tall_r * tiles_c;
            if (nb8 >= 512) {  // enough tall tiles for every CU to have a few
                const int grid = persistent_grid<fwd_mfma<BF, D, KS, false, 8>>(nb8, G8::NT);
                ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_mfma", st);
                if (!kNarrow && a.s.H % G8::TH == 0 && a.s.W % G8::TW == 0)
                    hipLaunchKernelGGL((fwd_mfma<BF, D, KS, false, 8, !kNarrow>), dim3(grid), dim3(G8::NT), 0,
                                       st, a, tall_r, tiles_c, (int)nb8, Runs{0, 0});
                else
                    hipLaunchKernelGGL((fwd_mfma<BF, D, KS, false, 8>), dim3(grid), dim3(G8::NT), 0, st, a,
                                       tall_r, tiles_c, (int)nb8, Runs{0, 0});
                return check_launch("enatten2d_fwd");
            }
        }
        if constexpr (kFwd2TallBuilt<D, KS>) {
            using G8 = Geo<D, KS, 8>;
            const int tall_r = (a.s.H + G8::TH - 1) / G8::TH;
            const int64_t nb8 = (int64_t)a.s.B * a.s.N * tall_r * tiles_c;
            if (nb8 >= 256) {  // a tile for every CU
                const int grid = persistent_grid<fwd2_mfma<BF, D, KS, 8>>(nb8, G8::NT);
                ProfScope prof(ENATTEN_KERNEL_FWD, "fwd2_mfma", st);
                if (!kNarrow && a.s.H % G8::TH == 0 && a.s.W % G8::TW == 0)
                    hipLaunchKernelGGL((fwd2_mfma<BF, D, KS, 8, !kNarrow>), dim3(grid), dim3(G8::NT), 0, st, a,
                                       tall_r, tiles_c, (int)nb8);
                else
                    hipLaunchKernelGGL((fwd2_mfma<BF, D, KS, 8>), dim3(grid), dim3(G8::NT), 0, st, a, tall_r,
                                       tiles_c, (int)nb8);
                return check_launch("enatten2d_fwd");
            }
        }
        if constexpr (kFwd2Built<D, KS>) {
            const int grid = persistent_grid<fwd2_mfma<BF, D, KS>>(nb);
            if (nb >= 2 * 256 || !fits<D, KS>()) {  // two workgroups for each of the 256 CUs
                ProfScope prof(ENATTEN_KERNEL_FWD, "fwd2_mfma", st);
                if (!kNarrow && a.s.H % G::TH == 0 && a.s.W % G::TW == 0)
                    hipLaunchKernelGGL((fwd2_mfma<BF, D, KS, 4, !kNarrow>), dim3(grid), dim3(256), 0, st, a,
                                       tiles_r, tiles_c, (int)nb);
                else
                    hipLaunchKernelGGL((fwd2_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, tiles_r,
                                       tiles_c, (int)nb);
                return check_launch("enatten2d_fwd");
            }
        }
        if constexpr (fits<D, KS>()) {
            const int grid = persistent_grid<fwd_mfma<BF, D, KS, false>>(nb);
            ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_mfma", st);
            const bool full = !kNarrow && a.s.H % G::TH == 0 && a.s.W % G::TW == 0;
            if (roll_pays<D>(nb, grid)) {
                if (full)
                    hipLaunchKernelGGL((fwd_mfma<BF, D, KS, kRollBuilt<D>, 4, !kNarrow>), dim3(grid), dim3(256),
                                       0, st, a, tiles_r, tiles_c, (int)nb, plan_runs(nb, grid, tiles_r));
                else
                    hipLaunchKernelGGL((fwd_mfma<BF, D, KS, kRollBuilt<D>>), dim3(grid), dim3(256), 0,
                                       st, a, tiles_r, tiles_c, (int)nb, plan_runs(nb, grid, tiles_r));
            } else if (full) {
                hipLaunchKernelGGL((fwd_mfma<BF, D, KS, false, 4, !kNarrow>), dim3(grid), dim3(256), 0, st, a,
                                   tiles_r, tiles_c, (int)nb, Runs{0, 0});
            } else {
                hipLaunchKernelGGL((fwd_mfma<BF, D, KS, false>), dim3(grid), dim3(256), 0, st, a,
                                   tiles_r, tiles_c, (int)nb, Runs{0, 0});
            }
        }
        return check_launch("enatten2d_fwd");
    } else {
        set_error("no matrix-core kernel for head_dim %d, kernel_size %d", D, KS);
        return ENATTEN_EUNSUPPORTED;
    }
}

// Where the FULL form of bwd_dq2_mfma is used: at head_dim 128 it was measured faster with
// kernel_size 7 and 11 (B4 N4 128x128: 76.7 -> 68.2 and 184.7 -> 173.2 us) and slower with 9
// and 13 (82.4 -> 84.4, and 167.5 -> 214.7 with the 16x8 tiles: what those two spill moves
// into their inner loops); at head_dim 64 faster (k11 76.2 -> 73.9, k13 76.2 -> 75.6).
template <int D, int KS>
constexpr bool kDq2Full = !kNarrow && (D != 128 || KS == 7 || KS == 11);

template <bool BF, int D, int KS>
int bwd_launch(const BwdArgs &a, int path, hipStream_t st) {
    if constexpr (kBuilt<D, KS>) {
        using G = Geo<D, KS>;
        const int tiles_r = (a.s.H + G::TH - 1) / G::TH, tiles_c = (a.s.W + G::TW - 1) / G::TW;
        const int64_t nb = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
        // inner tiles (no key or query within reach of the border) and frame
        TileSet ts;
        ts.tiles_r = tiles_r; ts.tiles_c = tiles_c;
        // (tile row tr, keys 8 tr .. 8 tr + 7, is inner when no query with a clamped window
        // attends to its keys: the queries of rows 0 .. k/2 - 1 reach the keys of rows 0 .. k - 1,
        // so 8 tr >= k, and 8 tr + 7 <= H - 1 - k at the other end)
        ts.ir0 = (KS + 7) / 8; ts.ic0 = (KS + 7) / 8;
        ts.ni_r = (a.s.H - KS) / 8 - ts.ir0; ts.ni_c = (a.s.W - KS) / 8 - ts.ic0;
        if (ts.ni_r <= 0 || ts.ni_c <= 0 || kDkdvFrameOnly<D, KS>) {
            ts.ir0 = tiles_r; ts.ic0 = 0; ts.ni_r = 0; ts.ni_c = 0;
        }
        const int64_t slabs = (int64_t)a.s.B * a.s.N;
        const int64_t n_inner = slabs * ts.ni_r * ts.ni_c, n_frame = nb - n_inner;

        // The fused backward wherever it is built (fused_bwd_supported): 5-25% faster than the
        // two passes at every size measured, from B64 N16 8x8 (45.7 against 47.3 us) and B4 N4
        // 32x32 (14.8 against 24.1) to B16 N8 128x128 (938 against 1174).
        if (!split_forced(path) && fused_bwd_supported(a)) {
            const int rc = launch_bwd_fused(a, BF, ts, nb, st);
            return rc ? rc : check_launch("enatten2d_bwd");
        }

        // The one-pass backward (head_dim 32, and 64 with kernel_size 3; na2d_mfma_onepass.hip).
        // At these head dims the passes are bound by per-tile latency, not by HBM, so reading
        // the inputs once only pays where the two passes are at their worst: images that are
        // (nearly) all border tiles, which the dK/dV pass walks block by block and the one-pass
        // kernel serves from its one staged block.  Measured on a settled GPU, backward kernels,
        // one pass vs two (us, bf16, head_dim 32, kernel_size 7): B8 N16 14x14 17.2 vs 13.2;
        // B8 N8 28x28 24.9 vs 24.8; B8 N4 40x40 22.0 vs 16.1 (9 of 25 tiles inner); B8 N4 56x56
        // 32.6 vs 26.4; B8 N2 112x112 51.4 vs 42.8.  The whole step replayed as a graph, where
        // one launch less counts: 14x14 30.3 vs 29.0, 28x28 39.2 vs 40.7, 40x40 37.8 vs 32.9,
        // 56x56 52.7 vs 49.0.  So it is the default only where at most one tile in eight is an
        // inner tile (level with the two passes there, one launch less);
        // ENATTEN_PATH_MFMA_FUSED forces it wherever it is built.
        if (!split_forced(path) && onepass_bwd_supported(a) &&
            (path == ENATTEN_PATH_MFMA_FUSED || 8 * n_inner <= nb)) {
            const int rc = launch_bwd_onepass(a, BF, ts, nb, st);
            return rc ? rc : check_launch("enatten2d_bwd");
        }

        bool dq_done = false;
        if constexpr (kDq2TallBuilt<D, KS>) {
            using G8 = Geo<D, KS, 8>;
            TileSet tall = ts;  // only the tile counts are used by this pass
            tall.tiles_r = (a.s.H + G8::TH - 1) / G8::TH;
            const int64_t nb8 = slabs * tall.tiles_r * tiles_c;
            if (nb8 >= 256) {
                const int grid = persistent_grid<bwd_dq2_mfma<BF, D, KS, 8>>(nb8, G8::NT);
                ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq2_mfma", st);
                if (kDq2Full<D, KS> && a.s.H % G8::TH == 0 && a.s.W % G8::TW == 0)
                    hipLaunchKernelGGL((bwd_dq2_mfma<BF, D, KS, 8, kDq2Full<D, KS>>), dim3(grid), dim3(G8::NT), 0,
                                       st, a, tall, (int)nb8);
                else
                    hipLaunchKernelGGL((bwd_dq2_mfma<BF, D, KS, 8>), dim3(grid), dim3(G8::NT), 0, st, a, tall,
                                       (int)nb8);
                dq_done = true;
            }
        }
        if constexpr (kDq2Built<D, KS>) {
            if (!dq_done) {
                const int grid = persistent_grid<bwd_dq2_mfma<BF, D, KS>>(nb);
                ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq2_mfma", st);
                if (kDq2Full<D, KS> && a.s.H % G::TH == 0 && a.s.W % G::TW == 0)
                    hipLaunchKernelGGL((bwd_dq2_mfma<BF, D, KS, 4, kDq2Full<D, KS>>), dim3(grid), dim3(256), 0, st,
                                       a, ts, (int)nb);
                else
                    hipLaunchKernelGGL((bwd_dq2_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, ts, (int)nb);
                dq_done = true;
            }
        } else if constexpr (kTallDqBuilt<D, KS>) {
            using G8 = Geo<D, KS, 8>;
            TileSet tall = ts;  // only the tile counts are used by this pass
            tall.tiles_r = (a.s.H + G8::TH - 1) / G8::TH;
            const int64_t nb8 = slabs * tall.tiles_r * tiles_c;
            if (nb8 >= 512) {
                const int grid = persistent_grid<bwd_dq_mfma<BF, D, KS, false, false, 8>>(nb8, G8::NT);
                ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_mfma", st);
                if (!kNarrow && a.s.H % G8::TH == 0 && a.s.W % G8::TW == 0)
                    hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, false, 8, !kNarrow>), dim3(grid),
                                       dim3(G8::NT), 0, st, a, tall, (int)nb8, Runs{0, 0});
                else
                    hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, false, 8>), dim3(grid), dim3(G8::NT),
                                       0, st, a, tall, (int)nb8, Runs{0, 0});
                dq_done = true;
            }
        }
        if constexpr (fits<D, KS>()) if (!dq_done) {
            const int grid = persistent_grid<bwd_dq_mfma<BF, D, KS, false, false>>(nb);
            ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_mfma", st);
            const bool full = !kNarrow && a.s.H % G::TH == 0 && a.s.W % G::TW == 0;
            if (roll_pays<D>(nb, grid)) {
                if (full)
                    hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, kRollBuilt<D>, 4, !kNarrow>), dim3(grid),
                                       dim3(256), 0, st, a, ts, (int)nb, plan_runs(nb, grid, tiles_r));
                else
                    hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, kRollBuilt<D>>), dim3(grid),
                                       dim3(256), 0, st, a, ts, (int)nb, plan_runs(nb, grid, tiles_r));
            } else if (full) {
                hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, false, 4, !kNarrow>), dim3(grid), dim3(256), 0,
                                   st, a, ts, (int)nb, Runs{0, 0});
            } else {
                hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS, false, false>), dim3(grid), dim3(256), 0,
                                   st, a, ts, (int)nb, Runs{0, 0});
            }
        }
        {
            // Share the resident workgroups between the two bodies so that they end together.
            // `cost` is a frame tile's time in inner tiles (measured): 2 at head_dim 64 (1.68 with
            // the frame body's larger blocks), 2.5 at head_dim 32 (against 2: B8 N2 112x112 k7
            // 28.7 -> 27.1 us, B8 N4 56x56 20.8 -> 18.6, B4 N4 128x128 k5 27.1 -> 25.4, k3 23.1 ->
            // 21.5; 2-4% slower at 96x96 and 256x256 k7), kFrameCost128 at head_dim 128.
            constexpr int SP = kDkdvSplit<D, KS>, NT = Geo<D, KS, 4, SP>::NT;
            const double cost = D >= 128 ? kFrameCost128<KS> : kFrameKS<D, KS, SP> != KS ? 1.68 : D == 32 ? 2.5 : 2.0;
            const int grid = persistent_grid<bwd_dkdv_mfma<BF, D, KS, false, SP>>(nb, NT);
            int inner_blocks = 0, dyn = 0;
            if (n_frame == 0) {
                inner_blocks = grid;
            } else if (n_inner > 0 && kRollBuilt<D>) {
                // With the column walk the busiest inner workgroup's walk is a staircase in the
                // number of inner workgroups (plan_runs), and a share in proportion to the work
                // lands anywhere on a step.  So every split is tried: the fewest inner
                // workgroups among those whose longer side is shortest.
                double best = 1e30;
                const int64_t per_f = (n_frame + 7) / 8, per_i = (n_inner + 7) / 8;
                for (int ib = 8; ib <= grid - 8 && ib <= per_i * 8; ib += 8) {
                    double walk;
                    if (roll_pays<D>(n_inner, ib)) {
                        plan_runs(n_inner, ib, ts.ni_r, &walk);
                    } else {
                        const int64_t slots_i = ib / 8;
                        walk = 2.0 * (double)((per_i + slots_i - 1) / slots_i);
                    }
                    const int64_t slots_f = (grid - ib) / 8;
                    const double frame = 2.0 * cost * (double)((per_f + slots_f - 1) / slots_f);
                    const double t = walk > frame ? walk : frame;
                    if (t < best) {
                        best = t;
                        inner_blocks = ib;
                    }
                }
                if (inner_blocks == 0) inner_blocks = 8;
                // The other way to share: every workgroup walks inner tiles (the shortest walk
                // there is) and then takes frame tiles from a counter as it becomes free.  The
                // frame tiles then run at the end, next to no inner tile and in no XCD's order,
                // which costs where the static split is already even; it is taken where the
                // staircase leaves the static split 7% or more behind (B4 N4 128x128 k7: 154.6 ->
                // 135.4 us; measured 4-9% slower at k9 and at 256x256 and 96x96 k7, where it is
                // not taken).
                if (a.zinv != nullptr) {
                    int all = grid;
                    if (all > per_i * 8) all = (int)(per_i * 8);
                    double walk;
                    if (roll_pays<D>(n_inner, all)) {
                        plan_runs(n_inner, all, ts.ni_r, &walk);
                    } else {
                        const int64_t slots_i = all / 8;
                        walk = 2.0 * (double)((per_i + slots_i - 1) / slots_i);
                    }
                    const double t_dyn = walk + 2.0 * cost * ((double)n_frame / grid + 1.0);
                    if (t_dyn < 0.93 * best) {
                        dyn = 1;
                        inner_blocks = all;
                    }
                }
            } else if (n_inner > 0) {
                const double f = (double)n_inner / ((double)n_inner + cost * (double)n_frame);
                inner_blocks = (int)(f * grid / 8.0 + 0.5) * 8;
                if (inner_blocks < 8) inner_blocks = 8;
                if (inner_blocks > grid - 8) inner_blocks = grid - 8;
                if (inner_blocks > (n_inner + 7) / 8 * 8) inner_blocks = (int)((n_inner + 7) / 8 * 8);
            }
            if (path == ENATTEN_PATH_MFMA_SPLIT_QUEUE && a.zinv != nullptr && n_frame > 0 && !dyn) {
                dyn = 1;
                const int64_t all = (n_inner + 7) / 8 * 8;
                inner_blocks = all < grid ? (int)all : grid;
            }
            ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd_dkdv_mfma", st);
            if (inner_blocks > 0 && roll_pays<D>(n_inner, inner_blocks))
                hipLaunchKernelGGL((bwd_dkdv_mfma<BF, D, KS, kRollBuilt<D>, SP>), dim3(grid), dim3(NT),
                                   0, st, a, ts, (int)n_inner, (int)n_frame, inner_blocks,
                                   plan_runs(n_inner, inner_blocks, ts.ni_r), dyn);
            else
                hipLaunchKernelGGL((bwd_dkdv_mfma<BF, D, KS, false, SP>), dim3(grid), dim3(NT), 0, st,
                                   a, ts, (int)n_inner, (int)n_frame, inner_blocks, Runs{0, 0}, dyn);
        }
        return check_launch("enatten2d_bwd");
    } else {
        set_error("no matrix-core kernel for head_dim %d, kernel_size %d", D, KS);
        return ENATTEN_EUNSUPPORTED;
    }
}

#define ENATTEN_BY_KS(FN, BF, D, ARGS, ...)                      \
    switch ((ARGS).s.kh) {                                       \
        case 3: return FN<BF, D, 3>(ARGS, __VA_ARGS__);          \
        case 5: return FN<BF, D, 5>(ARGS, __VA_ARGS__);          \
        case 7: return FN<BF, D, 7>(ARGS, __VA_ARGS__);          \
        case 9: return FN<BF, D, 9>(ARGS, __VA_ARGS__);          \
        case 11: return FN<BF, D, 11>(ARGS, __VA_ARGS__);        \
        case 13: return FN<BF, D, 13>(ARGS, __VA_ARGS__);        \
    }

// A head dim that is a multiple of 8 runs on the kernels built for the next of 32, 64 and
// 128: their LDS rows carry zeros in the channels the tensor does not have (zero_row,
// HaloPlan::on, load_row_chunks) and the stores leave those channels out (store_token).
constexpr int built_dim(int D) { return D <= 32 ? 32 : D <= 64 ? 64 : 128; }

#define ENATTEN_BY_D(FN, BF, ARGS, ...)                                  \
    switch (built_dim((ARGS).s.D)) {                                     \
        case 32: ENATTEN_BY_KS(FN, BF, 32, ARGS, __VA_ARGS__) break;     \
        case 64: ENATTEN_BY_KS(FN, BF, 64, ARGS, __VA_ARGS__) break;     \
        case 128: ENATTEN_BY_KS(FN, BF, 128, ARGS, __VA_ARGS__) break;   \
    }

bool fits_rt(int D, int ks) {
    const int rows = (8 + ks - 1) * (8 + ks - 1) + 1;
    // two halos of an 8x8 tile, or (head_dim 128) one halo for the kernels that stage one at a time
    return (size_t)2 * rows * (D + 8) * 2 + (size_t)rows * 8 <= 160 * 1024 ||
           (D == 128 && (size_t)rows * (D + 8) * 2 + 1024 <= 160 * 1024);
}

// The launchers' common body: tensors whose rows the 16-byte loads cannot take go to the
// general kernels, everything else to the kernel built for its head dim and kernel size.
int fwd_dispatch(const FwdArgs &a, int dtype, hipStream_t st) {
    if (!layout_ok(a.q) || !layout_ok(a.k) || !layout_ok(a.v) || !layout_ok(a.o))
        return launch_fwd_simt(a, dtype, st);  // 16-byte loads need aligned rows
    if (dtype == ENATTEN_BF16) {
        ENATTEN_BY_D(fwd_launch, true, a, st)
    } else {
        ENATTEN_BY_D(fwd_launch, false, a, st)
    }
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

int bwd_dispatch(const BwdArgs &a, int dtype, int path, hipStream_t st) {
    auto al = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    const bool grads_ok = a.gsb % 8 == 0 && a.gsn % 8 == 0 && a.gsh % 8 == 0 && a.gsw % 8 == 0;
    if (!layout_ok(a.q) || !layout_ok(a.k) || !layout_ok(a.v) || !layout_ok(a.o) ||
        !layout_ok(a.d_o) || !al(a.dq) || !al(a.dk) || !al(a.dv) || !grads_ok ||
        a.s.H >= 32768 || a.s.W >= 32768)  // (the dK/dV pass keeps window starts in 16 bits)
        return launch_bwd_simt(a, dtype, st);
    if (dtype == ENATTEN_BF16) {
        ENATTEN_BY_D(bwd_launch, true, a, path, st)
    } else {
        ENATTEN_BY_D(bwd_launch, false, a, path, st)
    }
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace
}  // namespace enatten
