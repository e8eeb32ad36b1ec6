// Fused backward of 2D neighborhood attention on the matrix cores of gfx950:
// dQ, dK and dV of an 8x8 tile of pixels from ONE staging of the tile's
// (8+k-1)^2 block of q, k, v and dO, so that the backward reads each input once
// (the two passes of na2d_mfma_kernels.h read them twice).
//
// A workgroup is eight waves around one copy of the block in LDS (all four
// tensors, which is why only one workgroup fits a CU):
//   waves 0-3  query side: dQ of their 4x4 queries over the keys of the block
//              (e_natten/triton.py:383-398 per query);
//   waves 4-7  key side: dK, dV of their 4x4 keys over the queries of the block
//              (the inverse neighbourhood of e_natten/pytorch.py:13-23, :261-288).
// Both sides recompute P from the saved log-sum-exp.  delta = dO . O of the block's
// queries is formed while the block is written to LDS (the forward output is read
// for this and for nothing else).  The MFMA operand layouts, the token numbering
// and the transposing LDS reads are those of na2d_mfma_kernels.h.
//
// The block of the tile at (r0, c0) is the pixels [r0 - k/2, r0 + 8 + k/2) x
// [c0 - k/2, c0 + 8 + k/2); with image sides that are multiples of 8 it holds
// every key a query of the tile attends to and every query that attends to a key
// of the tile, also beside the border (positions outside the image are staged as
// copies of the nearest pixel and masked).  Workgroups walk down the columns of an
// image, and the k-1 block rows that consecutive tiles share stay in LDS (image
// row y in row slot (y + k/2) % HR): a step stages 8 new rows.
//
// The kernel is persistent like the others: the next tile's rows travel from HBM
// into registers while the current tile is computed out of LDS.

#include "na2d_mfma.h"

namespace enatten {
namespace {

template <int D, int KS>
struct FGeo {
    using G = Geo<D, KS>;
    static constexpr int NT = 512;                        // threads per workgroup
    // Staging is shared unevenly: the key side has more arithmetic per tile, so the
    // query-side waves move five sixths of a step and the key-side waves the rest
    // (issuing a load blocks a wave for as long as some of its arithmetic takes).
    static constexpr int RPH = NT / 2 / G::CPR;           // block pixels per pass and side
    static constexpr int BR = 8;                          // block rows staged per step
    static constexpr int passes(int nrows) { return (nrows * G::HC + RPH - 1) / RPH; }
    static constexpr int q_passes(int nrows) {
        return passes(nrows) - (passes(nrows) / 6 > 1 ? passes(nrows) / 6 : 1);
    }
    static constexpr int NL = q_passes(BR);               // chunks per thread and tensor (query side)
    // Key side beside the border: the queries that attend to a wave's 4x4 keys
    // span up to SW + k/2 rows and columns there.
    static constexpr int SWB = G::SW + KS / 2;
    static constexpr size_t LDS_BYTES = (size_t)4 * G::ROWS * G::PITCH * sizeof(short) +
                                        (size_t)G::ROWS * sizeof(float2) + 4 * 64 * sizeof(int);
    static constexpr bool FITS = LDS_BYTES <= 160 * 1024 && G::HR - BR <= BR && SWB <= 16 &&
                                 SWB <= G::HR;
};

template <int NL>
struct Chunks {
    u32x4 v[NL];
};

// ok ? x : -inf as bit arithmetic.  Written as a conditional expression, the compiler
// moves the LDS read that feeds x under a branch on ok (one branch per logit).
__device__ __forceinline__ float keep_or_ninf(float x, bool ok) {
    const int m = ok ? -1 : 0;
    return __int_as_float((__float_as_int(x) & m) | ((int)0xff800000 & ~m));
}
template <bool BF, int D, int KS>
__global__ __launch_bounds__(512) void bwd_fused_mfma(BwdArgs a, TileSet ts, int ntiles) {
    using G = Geo<D, KS>;
    using F = FGeo<D, KS>;
    constexpr int HALF = KS / 2;
    __shared__ __attribute__((aligned(16))) short lds_q[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];
    // (log-sum-exp * log2(e), scale * dO . O) per staged query.  dS is formed with the softmax
    // scale in it, p * (scale * dP - scale * delta): one fused multiply-add where the difference
    // was one subtraction, and dQ and dK leave their accumulators without 32 multiplications each.
    __shared__ float2 lds_stat[G::ROWS];
    // per key-side wave, for a tile beside a border: LDS row | region row << 16 | region
    // column << 20 of each of its 64 query numbers
    __shared__ int lds_qtab[4 * 64];

    const Shape &s = a.s;
    // One contiguous run of column-major tiles per workgroup, all of the same length: a tile
    // beside a border costs about as much as an inner one since its key side runs the
    // unrolled body too (with run weights border : inner of 8:7, 16:15, 32:31 and 1:1 the
    // kernel takes 130.5, 128.6, 128.8 and 127.5 us at B4 N4 128x128), and runs of equal
    // length keep the workgroups of an XCD on neighbouring columns at the same height
    // where a run is one column.
    Sched sc;
    int deal_ncols = 0, deal_lo = 0, seg_end = 0, deal_round = 0;  // columns dealt in rounds, see below
    {
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
        const int per = (ntiles + 7) >> 3;
        const int lo = xcd * per, hi = max(min(ntiles, lo + per), lo);
        sc.t = lo + (int)((long long)(hi - lo) * slot / slots);
        sc.t_end = lo + (int)((long long)(hi - lo) * (slot + 1) / slots);
        sc.step = 1;
        // Where an XCD has two or more whole columns per workgroup, a contiguous run would
        // put its workgroups on columns that are never adjacent at the same time, and the
        // block columns that neighbouring tiles share would all come from HBM.  The XCD's
        // columns are then dealt in rounds instead: in round r workgroup `slot` walks column
        // r * slots + (slot + 2r) % slots, so that at any time the workgroups are on
        // neighbouring columns at the same height, and the rotation by 2r spreads the dearer
        // first and last columns of the images over the workgroups (B8 N8 128x128: 617 ->
        // 475 us; B4 N4 256x256: 599 -> 511).  The columns that do not fill a round are
        // shared out as one more contiguous run per workgroup.  (Columns cut into parts to
        // make rounds where there are fewer were measured slower, B2 N4 160x160: 113 -> 122 us.)
        if (per % ts.tiles_r == 0 && hi - lo == per && per / ts.tiles_r >= 2 * slots) {
            deal_ncols = per / ts.tiles_r;
            deal_lo = lo;
            sc.t = lo + slot * ts.tiles_r;  // r = 0: column `slot`
            seg_end = sc.t + ts.tiles_r;
            sc.t_end = hi;
        }
    }
    if (sc.t >= sc.t_end) return;
    // the tile after t in this workgroup's walk, or sc.t_end
    auto tile_after = [&](int t, int &round) __attribute__((always_inline)) {
        if (deal_ncols == 0 || t + 1 < seg_end) return t + 1;
        const int slots = gridDim.x >> 3, slot = blockIdx.x >> 3;
        round++;
        const int full = deal_ncols / slots;  // rounds in which every workgroup has a column
        if (round < full) {
            const int t0 = deal_lo + (round * slots + (slot + 2 * round) % slots) * ts.tiles_r;
            seg_end = t0 + ts.tiles_r;
            return t0;
        }
        if (round == full) {
            const int rest_lo = deal_lo + full * slots * ts.tiles_r, rest = sc.t_end - rest_lo;
            const int t0 = rest_lo + (int)((long long)rest * slot / slots);
            seg_end = rest_lo + (int)((long long)rest * (slot + 1) / slots);
            if (t0 < seg_end) return t0;
        }
        return sc.t_end;
    };
    const int tid = threadIdx.x;
    if (tid < G::CPR) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4 *>(lds_q + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_g + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_k + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_v + G::ZROW * G::PITCH + tid * 8) = z;
    }
    if (tid == 0) lds_stat[G::ZROW] = make_float2(0.f, 0.f);

    // the wave number through readfirstlane, so that the compiler knows it is uniform:
    // the role branch is then a scalar branch and per-wave values live in SGPRs
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63;
    const int role = wave >> 2, w = wave & 3;
    const float sc2 = s.scale * kLog2e;

    // ---- staging: a step moves BR rows x HC columns of the block, all five tensors.
    // Chunk i of this thread is channel chunk tid % CPR of pixel tid / CPR + i * RP of
    // the step (row-major).  Every tensor comes with its own row and pixel strides.
    int stid = tid;  // laundered once per tile, see the tile loop
    auto ch8_of = [&]() __attribute__((always_inline)) { return (stid % G::CPR) * 8; };
    Chunks<F::NL> qst, gst, kst, vst, ost;
    float lse_st = 0.f;
    // Pixel number (row-major inside the step) of chunk i of this thread, or -1: a
    // step of NR rows has NR*HC pixels; the query-side waves take the first
    // q_passes(NR) * RPH of them, the key-side waves the rest.
    auto step_pixel = [&](int i, auto nr, int side) __attribute__((always_inline)) {
        constexpr int NR = decltype(nr)::value;
        constexpr int QP = F::q_passes(NR), KP = F::passes(NR) - QP;
        const int mine = side == 0 ? QP : KP;
        const int pix = (side == 0 ? 0 : QP * F::RPH) + (stid & (F::NT / 2 - 1)) / G::CPR + i * F::RPH;
        // (where the passes cover the step exactly, the bound is known when compiling)
        constexpr bool EXACT = (NR * G::HC) % F::RPH == 0;
        return (i < mine && (EXACT || pix < NR * G::HC)) ? pix : -1;
    };
    // NR (a compile-time constant: BR, or HR - BR for the rest of a whole block) rows
    // from y0 on, HC columns from bc on, of one image; positions outside the image
    // take the nearest pixel.  The offsets are formed anew for every tensor: kept,
    // they would hold registers through the math of a whole tile.
    // `side` (a compile-time 0 or 1) is the side of the calling wave: the key-side waves
    // then provably never touch the chunk registers beyond their share.
    auto fetch = [&](Chunks<F::NL> &reg, const View &vw, const char *base, int y0, int bc, auto nr,
                     auto side) __attribute__((always_inline)) {
        constexpr int NR = decltype(nr)::value;
        constexpr int SIDE = decltype(side)::value;
        constexpr int MINE = SIDE == 0 ? F::q_passes(NR) : F::passes(NR) - F::q_passes(NR);
        const unsigned sh2 = (unsigned)vw.sh * 2u, sw2 = (unsigned)vw.sw * 2u;
#pragma unroll
        for (int i = 0; i < MINE; i++) {
            const int pix = step_pixel(i, nr, SIDE);
            if (pix >= 0) {
                const int y = min(max(y0 + pix / G::HC, 0), s.H - 1);
                const int x = min(max(bc + pix % G::HC, 0), s.W - 1);
                const unsigned off = __umul24((unsigned)y, sh2) + __umul24((unsigned)x, sw2) +
                                     (unsigned)ch8_of() * 2u;
                reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off);
            }
        }
    };
    // The loads of a step are issued in five parts (one tensor each) spread over the
    // math of the current tile: a CU only takes so many vector loads at a time, and a
    // wave that waits at the queue with all of them at once does no math meanwhile.
    // The image that is being staged: the start of its (batch, head) slice in every tensor.
    // Kept per image, not formed per tile: the tensors' pointers and outer strides are then
    // only needed where a run crosses into another image.
    const char *img_q, *img_k, *img_v, *img_g, *img_o;
    const float *img_lse;
    auto set_image = [&](const Tile &tl) __attribute__((always_inline)) {
        img_q = reinterpret_cast<const char *>(image<short>(a.q, tl));
        img_k = reinterpret_cast<const char *>(image<short>(a.k, tl));
        img_v = reinterpret_cast<const char *>(image<short>(a.v, tl));
        img_g = reinterpret_cast<const char *>(image<short>(a.d_o, tl));
        img_o = reinterpret_cast<const char *>(image<short>(a.o, tl));
        img_lse = a.lse + ((int64_t)tl.bb * s.N + tl.nn) * s.H * (int64_t)s.W;
    };
    auto fetch_part = [&](int part, int y0, int bc, auto nr, auto side) __attribute__((always_inline)) {
        constexpr int NR = decltype(nr)::value;
        if (part == 0) {
            fetch(qst, a.q, img_q, y0, bc, nr, side);
            const int id = min(stid, NR * G::HC - 1);
            const int y = min(max(y0 + id / G::HC, 0), s.H - 1), x = min(max(bc + id % G::HC, 0), s.W - 1);
            lse_st = img_lse[y * s.W + x];
        } else if (part == 1) {
            fetch(kst, a.k, img_k, y0, bc, nr, side);
        } else if (part == 2) {
            fetch(vst, a.v, img_v, y0, bc, nr, side);
        } else if (part == 3) {
            fetch(gst, a.d_o, img_g, y0, bc, nr, side);
        } else {
            fetch(ost, a.o, img_o, y0, bc, nr, side);
        }
    };
    // registers -> LDS; image row y goes to row slot (y + HALF) % HR
    // dO . O of the chunks this thread staged (every lane of a pixel gets the pixel's sum)
    auto deltas_as = [&](float (&d)[F::NL], auto nr, auto side) __attribute__((always_inline)) {
        constexpr int NR = decltype(nr)::value;
        constexpr int SIDE = decltype(side)::value;
        constexpr int MINE = SIDE == 0 ? F::q_passes(NR) : F::passes(NR) - F::q_passes(NR);
#pragma unroll
        for (int i = 0; i < MINE; i++) d[i] = group_sum<G::CPR>(dot8<BF>(gst.v[i], ost.v[i]));
    };
    auto commit_as = [&](int y0, auto nr, auto side, const float (&dl)[F::NL]) __attribute__((always_inline)) {
        constexpr int NR = decltype(nr)::value;
        constexpr int SIDE = decltype(side)::value;
        constexpr int MINE = SIDE == 0 ? F::q_passes(NR) : F::passes(NR) - F::q_passes(NR);
        const int s0 = (y0 + HALF) % G::HR;
        auto lds_row = [&](int pr, int pc) __attribute__((always_inline)) {
            int slot = s0 + pr;
            slot = slot >= G::HR ? slot - G::HR : slot;
            return slot * G::HC + pc;
        };
#pragma unroll
        for (int i = 0; i < MINE; i++) {
            const float d = dl[i];
            const int pix = step_pixel(i, nr, SIDE);
            if (pix >= 0) {
                const int row = lds_row(pix / G::HC, pix % G::HC);
                const int e = G::chunk_at(row, stid % G::CPR);
                *reinterpret_cast<u32x4 *>(lds_q + e) = qst.v[i];
                *reinterpret_cast<u32x4 *>(lds_g + e) = gst.v[i];
                *reinterpret_cast<u32x4 *>(lds_k + e) = kst.v[i];
                *reinterpret_cast<u32x4 *>(lds_v + e) = vst.v[i];
                if (ch8_of() == 0) lds_stat[row].y = d * s.scale;
            }
        }
        if (stid < NR * G::HC) lds_stat[lds_row(stid / G::HC, stid % G::HC)].x = lse_st * kLog2e;
    };
    constexpr std::integral_constant<int, 0> kQuerySide{};
    constexpr std::integral_constant<int, 1> kKeySide{};
    // NR rows at once, not overlapped with anything (first tile of a workgroup, first
    // tile of a column).  The side is a per-wave value, i.e. a scalar branch, and everything a
    // side does with the rows it loads (dO . O, the writes to LDS) stays inside that side's
    // branch.  The compiler places the waits for loads per path of the program: a path that
    // loads as one side and consumes as the other exists for it, leaves loads pending behind
    // the stores of dQ / dK / dV, and made every wave wait for its stores at the top of the
    // next tile (s_waitcnt vmcnt(0) there; B4 N4 128x128: 122.2 -> 120.7 us, B8 N8: 445 -> 432).
    auto stage_now_as = [&](int y0, int bc, auto nr, auto side) __attribute__((always_inline)) {
#pragma unroll
        for (int part = 0; part < 5; part++) fetch_part(part, y0, bc, nr, side);
        float d[F::NL];
        deltas_as(d, nr, side);
        commit_as(y0, nr, side, d);
    };
    auto stage_now = [&](int y0, int bc, auto nr) __attribute__((always_inline)) {
        if (role == 0) stage_now_as(y0, bc, nr, kQuerySide);
        else stage_now_as(y0, bc, nr, kKeySide);
    };
    constexpr std::integral_constant<int, F::BR> kStep{};
    constexpr std::integral_constant<int, G::HR - F::BR> kRest{};

    Tile cur = tile_of_cm(sc.t, ts.tiles_r, ts.tiles_c, s.N);
    set_image(cur);
    stage_now(cur.r0 - HALF, cur.c0 - HALF, kStep);
    stage_now(cur.r0 - HALF + F::BR, cur.c0 - HALF, kRest);
    __syncthreads();
    const int n = l & 15, g = l >> 4;
    static_assert(G::SWC == 8 && G::SW == 8 && G::NK == G::NKP,
                  "the token -> LDS row arithmetic below is written for an 8x8 wave halo");
    for (;;) {
        // The thread number is laundered once per tile: the staging arithmetic that is
        // derived from it would otherwise be hoisted out of the loop and held in
        // registers that are not there.
        stid = tid;
        asm volatile("" : "+v"(stid));
        // The staging registers carry nothing from one tile to the next (they are
        // filled during a tile and written to LDS at its end): start every tile with
        // fresh ones, or the chunks that only the query side fills would count as
        // live through the key side's arithmetic.
        {
            Chunks<F::NL> fresh;
#pragma unroll
            for (int i = 0; i < F::NL; i++) asm volatile("" : "=v"(fresh.v[i]));
            qst = fresh; gst = fresh; kst = fresh; vst = fresh; ost = fresh;
        }
        int round_n = deal_round;
        int tn;
        bool more;
        Tile nxt = cur;
        if ((deal_ncols == 0 || sc.t + 1 < seg_end) && sc.t + 1 < sc.t_end && cur.r0 + 8 < s.H) {
            // the usual step, to the tile below in the same column: no divisions
            tn = sc.t + 1;
            more = true;
            nxt.r0 = cur.r0 + 8;
        } else {
            tn = tile_after(sc.t, round_n);
            more = tn < sc.t_end;
            if (more) nxt = tile_of_cm(tn, ts.tiles_r, ts.tiles_c, s.N);
        }
        // the tile below in the same image: its block shares k-1 rows with this one
        const bool below = more && nxt.bb == cur.bb && nxt.nn == cur.nn && nxt.c0 == cur.c0 &&
                           nxt.r0 == cur.r0 + 8;
        if (nxt.bb != cur.bb || nxt.nn != cur.nn) set_image(nxt);
        const int ny0 = below ? cur.r0 - HALF + G::HR : nxt.r0 - HALF;
        const int nbc = nxt.c0 - HALF;
        auto issue_as = [&](int part, auto side) __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            if (more) fetch_part(part, ny0, nbc, kStep, side);
            __builtin_amdgcn_sched_barrier(0);
        };

        // The end of a tile, per side: dO . O of the next step's rows (before the barrier: the
        // query side, which stages most of them, would wait there for the key side anyway), the
        // barrier after which no wave reads this tile's LDS any more, and the rows' way to LDS.
        auto finish_as = [&](auto side) __attribute__((always_inline)) {
            if (!more) {
                // (only the last tile of a workgroup comes here.  The explicit wait tells the
                // compiler that no load is pending on this path either: it does not know that
                // the loads were skipped under the same condition.)
                __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
                return;
            }
            float dnext[F::NL];
            deltas_as(dnext, kStep, side);
            __syncthreads();
            commit_as(ny0, kStep, side, dnext);
            if (!below) stage_now_as(ny0 + F::BR, nbc, kRest, side);
        };

        const int br = cur.r0 - HALF, bc = cur.c0 - HALF;
        const int rot = cur.r0 % G::HR;  // row slot of block row 0
        // LDS row of block position (r, c)
        auto block_row = [&](int r, int c) __attribute__((always_inline)) {
            int x = r + rot;
            x = x >= G::HR ? x - G::HR : x;
            return x * G::HC + c;
        };
        // Tokens of a wave's 8x8 halo with origin (orow, ocol) in the block: token
        // number tk is halo row tk / 8, column tk % 8.  All token numbers used below
        // have the form 8 * (a + bit) + c with a a compile-time even number, bit one
        // lane bit and c < 8, so the LDS row is one of two per-wave (scalar) row-slot
        // offsets plus a lane column: two or three vector instructions per address.
        int slot_of[G::SW];
        auto set_slots = [&](int orow) __attribute__((always_inline)) {
#pragma unroll
            for (int j = 0; j < G::SW; j++) {
                int x = orow + j + rot;
                x = x >= G::HR ? x - G::HR : x;
                slot_of[j] = x * G::HC;
            }
        };
        auto tok_row = [&](int a, int bit, int col) __attribute__((always_inline)) {
            return (bit ? slot_of[a + 1] : slot_of[a]) + col;
        };
        // this lane's pixel (query or key)
        const int py = cur.r0 + (w >> 1) * 4 + (n >> 2), px = cur.c0 + (w & 1) * 4 + (n & 3);
        const int prow = block_row(py - br, px - bc);
        auto out_token = [&]() __attribute__((always_inline)) {
            return (((int64_t)cur.bb * s.N + cur.nn) * s.H + py) * s.W + px;
        };
        const int tr = cur.r0 >> 3, tc = cur.c0 >> 3;
        const bool inner = tr >= ts.ir0 && tr < ts.ir0 + ts.ni_r && tc >= ts.ic0 && tc < ts.ic0 + ts.ni_c;

        if (role == 0) {
            auto issue = [&](int part) __attribute__((always_inline)) { issue_as(part, kQuerySide); };
            // ---- query side: this lane's query is column n of every product.  The
            // wave's keys are the (4+k-1)^2 pixels from the window start of its first
            // query row / column on.
            const int wy0 = cur.r0 + (w >> 1) * 4, wx0 = cur.c0 + (w & 1) * 4;
            const int sy0 = win_start(wy0, s.H, KS), sx0 = win_start(wx0, s.W, KS);
            const int orow = sy0 - br, ocol = sx0 - bc;
            const int dr = win_start(py, s.H, KS) - sy0, dc = win_start(px, s.W, KS) - sx0;
            set_slots(orow);
            s16x8 qreg[G::DS], greg[G::DS];
            {
                const typename G::ARow qp = G::a_row(lds_q, prow, g), gp = G::a_row(lds_g, prow, g);
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    qreg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(qp, ds));
                    greg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(gp, ds));
                }
            }
            const float2 mine = lds_stat[prow];
            const float lse2 = mine.x, delta_s = mine.y;
            s16x8 dsb[G::KSTEPS];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                if (mt < 4) issue(mt);
                const int row = tok_row(2 * mt, n >> 3, ocol + (n & 7));
                const typename G::ARow kp = G::a_row(lds_k, row, g), vp = G::a_row(lds_v, row, g);
                f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(kp, ds)), qreg[ds], cs);
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(vp, ds)), greg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    // key of accumulator row g*4+i: halo row 2*mt + g/2, column 4*(g%2) + i
                    const bool ok = ((unsigned)(2 * mt + (g >> 1) - dr) < (unsigned)KS) &
                                    ((unsigned)(4 * (g & 1) + i - dc) < (unsigned)KS);
                    const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - lse2 : -INFINITY);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * fmaf(cp[i], s.scale, -delta_s));
                }
            }
            issue(4);
            f32x4 dq[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                typename G::TRow kp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    kp[h] = G::t_row(lds_k, tok_row(4 * ks + 2 * h, g >> 1, ocol + 4 * (g & 1) + (n >> 2)), n);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    dq[mt] = mfma16<BF>(
                        cat(lds_read_tr(G::t_at(kp[0], mt)), lds_read_tr(G::t_at(kp[1], mt))), dsb[ks],
                        dq[mt]);
            }
            store_token<BF, D, false, true>(static_cast<short *>(a.dq) + out_token() * D, g, dq, 1.f, true);
            finish_as(kQuerySide);
        } else {
            auto issue = [&](int part) __attribute__((always_inline)) { issue_as(part, kKeySide); };
            // ---- key side: this lane's key is column n of every product
            // The unrolled key-side body, for at most 64 queries (4 row tiles of 16): P and dS
            // of all of them first, then dV and dK one after the other (one accumulator at a
            // time leaves the registers to the next tile's rows).  The caller says where the
            // queries are: arow(mt) is the LDS row of query mt*16 + n; stat(mt, i) and ok(mt, i)
            // are the statistics of query mt*16 + g*4 + i and whether it attends this lane's
            // key; trow(ks, h) is the LDS row of query ks*32 + h*16 + g*4 + n/4.
            auto key_body = [&](int krow_lds, int64_t tok, auto arow, auto stat, auto ok_fn, auto trow)
                                __attribute__((always_inline)) {
                s16x8 pb[G::KSTEPS], dsb[G::KSTEPS];
                {
                    s16x8 kreg[G::DS], vreg[G::DS];
                    {
                        const typename G::ARow kp = G::a_row(lds_k, krow_lds, g), vp = G::a_row(lds_v, krow_lds, g);
#pragma unroll
                        for (int ds = 0; ds < G::DS; ds++) {
                            kreg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(kp, ds));
                            vreg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(vp, ds));
                        }
                    }
#pragma unroll
                    for (int mt = 0; mt < G::MT; mt++) {
                        if (mt < 4) issue(mt);
                        f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
                        const int row = arow(mt);
                        const typename G::ARow qp = G::a_row(lds_q, row, g), gp = G::a_row(lds_g, row, g);
#pragma unroll
                        for (int ds = 0; ds < G::DS; ds++) {
                            cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(qp, ds)), kreg[ds], cs);
                            cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(gp, ds)), vreg[ds], cp);
                        }
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float2 st = stat(mt, i);
                            const float p = __builtin_amdgcn_exp2f(keep_or_ninf(cs[i] * sc2 - st.x, ok_fn(mt, i)));
                            pb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                            dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * fmaf(cp[i], s.scale, -st.y));
                        }
                    }
                }
                issue(4);
                auto second = [&](const short *lds_x, const s16x8 (&b)[G::KSTEPS], void *out, float mul)
                                  __attribute__((always_inline)) {
                    f32x4 acc[G::DT];
#pragma unroll
                    for (int mt = 0; mt < G::DT; mt++) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < G::KSTEPS; ks++) {
                        typename G::TRow xt[2];
#pragma unroll
                        for (int h = 0; h < 2; h++) xt[h] = G::t_row(lds_x, trow(ks, h), n);
#pragma unroll
                        for (int mt = 0; mt < G::DT; mt++)
                            acc[mt] = mfma16<BF>(
                                cat(lds_read_tr(G::t_at(xt[0], mt)), lds_read_tr(G::t_at(xt[1], mt))), b[ks],
                                acc[mt]);
                    }
                    store_token<BF, D, true, true>(static_cast<short *>(out) + tok * D, g, acc, mul, true);
                };
                second(lds_g, pb, a.dv, 1.f);
                second(lds_q, dsb, a.dk, 1.f);
            };
            const bool edge_r = tr == 0 || tr == ts.tiles_r - 1, edge_c = tc == 0 || tc == ts.tiles_c - 1;
            if (inner) {
                // Every window is centred: the queries are the (4+k-1)^2 pixels around the
                // wave's 4x4 keys, 8 to a row, and the mask depends on the lane only.
                const int ocol = (w & 1) * 4;
                set_slots((w >> 1) * 4);
                const int kyl = n >> 2, kxl = n & 3;
                key_body(
                    prow, out_token(),
                    [&](int mt) __attribute__((always_inline)) { return tok_row(2 * mt, n >> 3, ocol + (n & 7)); },
                    // queries of accumulator rows g*4 .. g*4+3: halo row 2*mt + g/2, columns
                    // 4*(g%2) .. +3, i.e. four consecutive LDS rows
                    [&](int mt, int i) __attribute__((always_inline)) {
                        return lds_stat[tok_row(2 * mt, g >> 1, ocol + 4 * (g & 1)) + i];
                    },
                    [&](int mt, int i) __attribute__((always_inline)) {
                        return ((unsigned)(2 * mt + (g >> 1) - kyl) < (unsigned)KS) &
                               ((unsigned)(4 * (g & 1) + i - kxl) < (unsigned)KS);
                    },
                    [&](int ks, int h) __attribute__((always_inline)) {
                        return tok_row(4 * ks + 2 * h, g >> 1, ocol + 4 * (g & 1) + (n >> 2));
                    });
            }
            // ---- key side of a tile beside a border; false if a wave has more queries than
            // the unrolled body serves.
            auto border_body = [&]() __attribute__((always_inline)) {
                // ---- key side of a tile beside a border.  The clamped windows put more
                // queries on the keys 3 and 4 pixels from a border and fewer on those beside
                // it: with 4x4 blocks of keys, the waves away from the border would have 10
                // rows (or columns, or both) of queries and the others 6, the same total as in
                // an inner tile but unevenly split.  So the waves take other sets of 16 keys:
                //  * beside one border, strips that run away from it, 8 x 2 beside the top or
                //    bottom and 2 x 8 beside the left or right: 10 x 6 queries per wave;
                //  * in a corner (written for the top left one, mirrored for the others): rows
                //    6-7 of the tile (6 x 10 queries); columns 6-7 of rows 0-5 and column 5 of
                //    rows 0-3 (8 x 7); columns 0-1 of rows 0-5 and column 2 of rows 0-3 (8 x 5);
                //    the rest (8 x 8).
                // Every wave then has at most the 64 queries that the unrolled body serves.
                int kyl, kxl;
                if (edge_r != edge_c) {
                    kyl = edge_r ? n >> 1 : 2 * w + (n >> 3);
                    kxl = edge_r ? 2 * w + (n & 1) : n & 7;
                } else {
                    if (w == 0) {
                        kyl = 6 + (n >> 3); kxl = n & 7;
                    } else if (w == 3) {
                        kyl = n < 2 ? 4 + n : n < 14 ? (n - 2) >> 1 : n - 10;
                        kxl = n < 2 ? 2 : n < 14 ? 3 + ((n - 2) & 1) : 5;
                    } else {
                        kyl = n < 12 ? n >> 1 : n - 12;
                        kxl = w == 1 ? (n < 12 ? 6 + (n & 1) : 5) : (n < 12 ? n & 1 : 2);
                    }
                    if (tr != 0) kyl = 7 - kyl;  // bottom corners
                    if (tc != 0) kxl = 7 - kxl;  // right corners
                }
                const int ky = cur.r0 + kyl, kx = cur.c0 + kxl;
                // the query rows / columns that attend any of the wave's keys: their bounding
                // box, from the 16 lanes' own ranges
                int r_lo = inv_lo(ky, KS), r_hi = inv_hi(ky, s.H, KS), c_lo = inv_lo(kx, KS), c_hi = inv_hi(kx, s.W, KS);
#pragma unroll
                for (int off = 1; off < 16; off <<= 1) {
                    r_lo = min(r_lo, __shfl_xor(r_lo, off, 64));
                    r_hi = max(r_hi, __shfl_xor(r_hi, off, 64));
                    c_lo = min(c_lo, __shfl_xor(c_lo, off, 64));
                    c_hi = max(c_hi, __shfl_xor(c_hi, off, 64));
                }
                const int qr0 = __builtin_amdgcn_readfirstlane(r_lo), qc0 = __builtin_amdgcn_readfirstlane(c_lo);
                const int nr = __builtin_amdgcn_readfirstlane(r_hi) - qr0;
                const int nc = __builtin_amdgcn_readfirstlane(c_hi) - qc0;
                const int nq = nr * nc;
                if (nq > G::NKP || nr > F::SWB || nc > F::SWB) return false;  // (not met; the general loop below serves it)
                const int orow = qr0 - br, ocol = qc0 - bc;
                const int magic = (65536 + nc - 1) / nc;  // tk * magic >> 16 == tk / nc for tk < 2048
                unsigned rmask = 0, cmask = 0;
#pragma unroll
                for (int r = 0; r < F::SWB; r++) {
                    const int qy = qr0 + r, qx = qc0 + r;
                    const bool oky = (r < nr) & ((unsigned)(ky - win_start(qy, s.H, KS)) < (unsigned)KS);
                    const bool okx = (r < nc) & ((unsigned)(kx - win_start(qx, s.W, KS)) < (unsigned)KS);
                    rmask |= (oky ? 1u : 0u) << r;
                    cmask |= (okx ? 1u : 0u) << r;
                }
                // Every lane works out where one query number lives; the wave reads the table
                // back wherever the body asks for a query (24 times per lane).  Numbers past
                // the region get the zero row and a row bit that no key has.
                int *qtab = lds_qtab + w * 64;
                {
                    const int r = (l * magic) >> 16, c = l - r * nc;
                    qtab[l] = l < nq ? block_row(orow + r, ocol + c) | (r << 16) | (c << 20)
                                     : (int)G::ZROW | (15 << 16);
                }
                auto ok_at = [&](int e) __attribute__((always_inline)) {
                    return ((rmask >> ((e >> 16) & 15)) & (cmask >> (e >> 20)) & 1u) != 0u;
                };
                key_body(
                    block_row(ky - br, kx - bc), (((int64_t)cur.bb * s.N + cur.nn) * s.H + ky) * s.W + kx,
                    [&](int mt) __attribute__((always_inline)) { return qtab[mt * 16 + n] & 0xffff; },
                    [&](int mt, int i) __attribute__((always_inline)) {
                        return lds_stat[qtab[mt * 16 + g * 4 + i] & 0xffff];
                    },
                    [&](int mt, int i) __attribute__((always_inline)) { return ok_at(qtab[mt * 16 + g * 4 + i]); },
                    [&](int ks, int h) __attribute__((always_inline)) {
                        return qtab[ks * 32 + h * 16 + g * 4 + (n >> 2)] & 0xffff;
                    });
                return true;
            };
            if (!inner && !border_body()) {
                // ---- the general key side, for a wave whose queries are more than the
                // unrolled body serves (no tile of an image with sides that are multiples of
                // 8 is known to need it).  4x4 blocks of keys; the set of queries that attend
                // to them is up to SW + k/2 wide per axis:
                // walk that region 32 queries at a time, with one bit per region row /
                // column telling whether that query row / column attends this lane's key
                // row / column.  The loop is rolled
                // (unrolled, the addresses of the whole region would be formed up front).
                const int kr0 = (w >> 1) * 4, kc0 = (w & 1) * 4, krn = 4, kcn = 4;
                const int ky = py, kx = px;
                const int krow_lds = prow;
                // query rows / columns that attend the block's key rows / columns
                const int qr0 = inv_lo(cur.r0 + kr0, KS), qc0 = inv_lo(cur.c0 + kc0, KS);
                const int nr = inv_hi(cur.r0 + kr0 + krn - 1, s.H, KS) - qr0;
                const int nc = inv_hi(cur.c0 + kc0 + kcn - 1, s.W, KS) - qc0;
                const int orow = qr0 - br, ocol = qc0 - bc;
                // the region's queries are numbered row-major, nc to a row
                const int nq = nr * nc, nks = (nq + 31) >> 5;
                const int magic = (65536 + nc - 1) / nc;  // tk * magic >> 16 == tk / nc for tk < 2048
                unsigned rmask = 0, cmask = 0;
#pragma unroll
                for (int r = 0; r < F::SWB; r++) {
                    const int qy = qr0 + r, qx = qc0 + r;
                    const bool oky = (r < nr) & ((unsigned)(ky - win_start(qy, s.H, KS)) < (unsigned)KS);
                    const bool okx = (r < nc) & ((unsigned)(kx - win_start(qx, s.W, KS)) < (unsigned)KS);
                    rmask |= (oky ? 1u : 0u) << r;
                    cmask |= (okx ? 1u : 0u) << r;
                }
                auto row_of = [&](int tk) __attribute__((always_inline)) {
                    const int r = (tk * magic) >> 16, c = tk - r * nc;
                    return tk < nq ? block_row(orow + r, ocol + c) : (int)G::ZROW;
                };
                auto ok_of = [&](int tk) __attribute__((always_inline)) {
                    const int r = (tk * magic) >> 16, c = tk - r * nc;
                    return (tk < nq) & (((rmask >> r) & (cmask >> c) & 1u) != 0u);
                };
                // this lane's key and value rows are read from LDS where they are used
                // (the registers do not hold them beside the two accumulators and the
                // next tile's rows)
                const int pkey = G::key(krow_lds), kvh = pkey >> 2;
                int kvoff = krow_lds * G::PITCH + ((g ^ (pkey & 3)) << 3);
                f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                    dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
                // (the next step's loads are issued around the loop, not in it: inside a
                // rolled loop their destination registers would have to be copied, which
                // means waiting for them)
                issue(0);
                issue(1);
#pragma unroll 1
                for (int ks = 0; ks < nks; ks++) {
                    asm volatile("" : "+v"(kvoff));  // keep their reads in the loop
                    const short *krow = lds_k + kvoff, *vrow = lds_v + kvoff;
                    s16x8 pb, dsb;
#pragma unroll
                    for (int m2 = 0; m2 < 2; m2++) {
                        const int mt = ks * 2 + m2;
                        const int row = row_of(mt * 16 + n);
                        const typename G::ARow qp = G::a_row(lds_q, row, g), gp = G::a_row(lds_g, row, g);
                        f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ds = 0; ds < G::DS; ds++) {
                            // the same logical chunk g + 4 * ds of the query row and of this
                            // lane's key row, each where its own row keeps it
                            cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(qp, ds)),
                                        *reinterpret_cast<const s16x8 *>(krow + ((ds ^ kvh) << 5)), cs);
                            cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(G::a_at(gp, ds)),
                                            *reinterpret_cast<const s16x8 *>(vrow + ((ds ^ kvh) << 5)), cp);
                        }
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const int tk = mt * 16 + g * 4 + i;  // query of accumulator row g*4+i
                            const float2 st = lds_stat[row_of(tk)];
                            const float p = __builtin_amdgcn_exp2f(keep_or_ninf(cs[i] * sc2 - st.x, ok_of(tk)));
                            pb[m2 * 4 + i] = cvt16<BF>(p);
                            dsb[m2 * 4 + i] = cvt16<BF>(p * fmaf(cp[i], s.scale, -st.y));
                        }
                    }
                    typename G::TRow qt[2], gt[2];
#pragma unroll
                    for (int h = 0; h < 2; h++) {
                        const int row = row_of(ks * 32 + h * 16 + g * 4 + (n >> 2));
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
                issue(2);
                issue(3);
                issue(4);
                const int64_t tok = (((int64_t)cur.bb * s.N + cur.nn) * s.H + ky) * s.W + kx;
                store_token<BF, D, true, true>(static_cast<short *>(a.dk) + tok * D, g, dk, 1.f, true);
                store_token<BF, D, true, true>(static_cast<short *>(a.dv) + tok * D, g, dv, 1.f, true);
            }
            finish_as(kKeySide);
        }

        if (!more) break;
        __syncthreads();
        cur = nxt;
        sc.t = tn;
        deal_round = round_n;
    }
}

template <bool BF, int D, int KS>
int fused_launch(const BwdArgs &a, const TileSet &ts, int64_t ntiles, hipStream_t st) {
    if constexpr (FGeo<D, KS>::FITS) {
        const int64_t per_xcd = (ntiles + 7) / 8;
        const int grid = (int)(8 * (per_xcd < 32 ? per_xcd : 32));  // one workgroup per CU
        ProfScope prof(ENATTEN_KERNEL_BWD_FUSED, "bwd_fused_mfma", st);
        hipLaunchKernelGGL((bwd_fused_mfma<BF, D, KS>), dim3(grid), dim3(512), 0, st, a, ts,
                           (int)ntiles);
        return ENATTEN_OK;
    } else {
        return ENATTEN_EUNSUPPORTED;
    }
}

}  // namespace

// The fused backward is built for head_dim 128 with kernel_size 5.  It needs image
// sides that are multiples of 8 (then the block of a tile holds everything the tile
// needs, also beside the border) and 32-bit byte offsets inside one image of every
// input (24-bit row and pixel strides are checked by layout_ok).
bool fused_bwd_supported(const BwdArgs &a) {
    auto small = [&](const View &v) {
        return ((int64_t)a.s.H * v.sh + (int64_t)a.s.W * v.sw + a.s.D) * 2 < ((int64_t)1 << 32);
    };
    return a.s.D == 128 && a.s.kh == 5 && a.s.kw == 5 && a.s.H % 8 == 0 && a.s.W % 8 == 0 &&
           a.grads_contiguous() &&
           small(a.q) && small(a.k) && small(a.v) && small(a.o) && small(a.d_o);
}

// dQ, dK, dV of all tiles in one launch.
int launch_bwd_fused(const BwdArgs &a, bool bf16, const TileSet &ts, int64_t ntiles,
                     hipStream_t st) {
    if (a.s.D == 128 && a.s.kh == 5) {
        if (bf16) return fused_launch<true, 128, 5>(a, ts, ntiles, st);
        return fused_launch<false, 128, 5>(a, ts, ntiles, st);
    }
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace enatten
