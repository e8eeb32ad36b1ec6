// One-pass backward of 2D neighborhood attention on the matrix cores of gfx950 for the
// configurations whose staged block of ALL four inputs fits LDS at least twice per CU
// (head_dim 32 with kernel_size 3, 5, 7; head_dim 64 with kernel_size 3): dQ, dK and dV of an
// 8x8 tile of pixels from one staging of the tile's (8+k-1)^2 block of q, k, v and dO, so
// that the backward reads every input once where the two passes of na2d_mfma_kernels.h read them
// twice (the reference's backward is one kernel too, e_natten/triton.py:304-423, with atomics
// where this one gathers over the inverse neighbourhood).
//
// A workgroup is four waves; each wave owns a 4x4 block of the tile and forms first dQ of
// its 16 pixels as queries over the keys of the block (e_natten/triton.py:383-398 per query),
// then dK and dV of the same 16 pixels as keys over the queries of the block that attend to
// them (the inverse neighbourhood of e_natten/pytorch.py:13-23, :261-288), all operands out
// of LDS.  delta = dO . O of every staged query is formed while the block is written to LDS
// (the forward output is read for this alone).  Operand layouts, token numbering and the
// transposing LDS reads are those of na2d_mfma_kernels.h; this is the 2D twin of bwd1d_fused_mfma.
//
// Tiles and blocks for any image with sides >= 8: tile origins are min(8 t, L - 8) on each
// axis (the last tile is shifted back to end with the image), and a pixel in the last 8 rows
// (columns) is written by the last tile of its column (row) of tiles only.  The block of a
// tile starts at clamp(origin - k/2, 0, L - (8+k-1)) (0 where the image is smaller than a
// block).  With k <= 8 it then holds every key that a pixel the tile writes attends to, and
// every query that attends to such a pixel: pixels within k of either border belong to the
// first or the last tile of the axis, whose blocks reach the border.

#include "na2d_mfma.h"

namespace enatten {
namespace {

template <int D, int KS>
struct OGeo {
    using G = Geo<D, KS>;
    static constexpr size_t LDS_BYTES =
        (size_t)4 * G::ROWS * G::PITCH * sizeof(short) + (size_t)G::ROWS * sizeof(float2);
    // built where LDS holds the block of two workgroups (two independent waves per SIMD) and
    // one thread per staged pixel carries its log-sum-exp
    static constexpr bool BUILT = (D == 32 || D == 64) && KS <= 7 && 2 * LDS_BYTES <= 160 * 1024 &&
                                  G::HR * G::HC <= 256;
};

// Tile t of an image (row-major over the tiles): origin shifted back at the far borders.
struct OTile {
    int bb, nn, r0, c0;
    bool last_r, last_c;
};
__device__ __forceinline__ OTile otile_of(int t, int tiles_r, int tiles_c, const Shape &s) {
    OTile tl;
    const int tc = t % tiles_c; t /= tiles_c;
    const int tr = t % tiles_r; t /= tiles_r;
    tl.c0 = min(tc * 8, s.W - 8);
    tl.r0 = min(tr * 8, s.H - 8);
    tl.last_c = tc == tiles_c - 1;
    tl.last_r = tr == tiles_r - 1;
    tl.bb = t / s.N; tl.nn = t % s.N;
    return tl;
}

template <bool BF, int D, int KS>
__global__ __launch_bounds__(256, 2) void bwd_onepass_mfma(BwdArgs a, TileSet ts, int ntiles) {
    using G = Geo<D, KS>;
    constexpr int HALF = KS / 2;
    __shared__ __attribute__((aligned(16))) short lds_q[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];
    __shared__ float2 lds_stat[G::ROWS];  // (log-sum-exp * log2(e), dO . O) per staged pixel

    const Shape &s = a.s;
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    zero_row<D, KS>(lds_q);
    zero_row<D, KS>(lds_g);
    zero_row<D, KS>(lds_k);
    zero_row<D, KS>(lds_v);
    if (threadIdx.x == 0) lds_stat[G::ZROW] = make_float2(0.f, 0.f);

    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n_lane = l & 15, g_lane = l >> 4;
    const float sc2 = s.scale * kLog2e;
    // origin of a tile's block in the image
    auto block_r = [&](const OTile &tl) __attribute__((always_inline)) {
        return min(max(tl.r0 - HALF, 0), max(s.H - G::HR, 0));
    };
    auto block_c = [&](const OTile &tl) __attribute__((always_inline)) {
        return min(max(tl.c0 - HALF, 0), max(s.W - G::HC, 0));
    };

    const HaloPlan<D, KS> plan = make_plan<D, KS>();
    HaloRegs<D, KS> qst, gst, kst, vst, ost;
    float lse_st = 0.f;
    auto img = [&](const View &vw, const OTile &tl) __attribute__((always_inline)) {
        return static_cast<const short *>(vw.ptr) + tl.bb * vw.sb + tl.nn * vw.sn;
    };
    // The next tile's rows travel in two parts: q and k (and the log-sum-exp) while this
    // tile's dQ is formed, v, dO and O when its arithmetic is over.  Loaded earlier (while dK
    // and dV are formed) they did not fit beside the accumulators at kernel_size 7 and at
    // head_dim 64: the compiler spilled 24 and 38 registers, freshly loaded rows among them,
    // each spill behind a wait for its load (B8 N2 112x112 d32 k7: 56.1 -> 53.3 us, B8 N8 28x28:
    // 27.2 -> 25.2, B8 N4 56x56 d64 k3: 31.2 -> 30.0; nothing is spilled now).
    auto prefetch_qk = [&](const OTile &tl) __attribute__((always_inline)) {
        const int br = block_r(tl), bc = block_c(tl);
        halo_fetch<D, KS>(qst, plan, img(a.q, tl), a.q.sh, a.q.sw, br, bc, s.H, s.W);
        halo_fetch<D, KS>(kst, plan, img(a.k, tl), a.k.sh, a.k.sw, br, bc, s.H, s.W);
        const int id = min((int)threadIdx.x, G::ZROW - 1);
        const int y = min(br + id / G::HC, s.H - 1), x = min(bc + id % G::HC, s.W - 1);
        lse_st = a.lse[(((int64_t)tl.bb * s.N + tl.nn) * s.H + y) * s.W + x];
    };
    auto prefetch_vgo = [&](const OTile &tl) __attribute__((always_inline)) {
        const int br = block_r(tl), bc = block_c(tl);
        halo_fetch<D, KS>(vst, plan, img(a.v, tl), a.v.sh, a.v.sw, br, bc, s.H, s.W);
        halo_fetch<D, KS>(gst, plan, img(a.d_o, tl), a.d_o.sh, a.d_o.sw, br, bc, s.H, s.W);
        halo_fetch<D, KS>(ost, plan, img(a.o, tl), a.o.sh, a.o.sw, br, bc, s.H, s.W);
    };

    OTile cur = otile_of(sc.t, ts.tiles_r, ts.tiles_c, s);
    prefetch_qk(cur);
    prefetch_vgo(cur);
    for (;;) {
        halo_commit<D, KS>(lds_q, plan, qst);
        halo_commit<D, KS>(lds_g, plan, gst);
        halo_commit<D, KS>(lds_k, plan, kst);
        halo_commit<D, KS>(lds_v, plan, vst);
#pragma unroll
        for (int i = 0; i < G::NL; i++) {
            const float d = group_sum<G::CPR>(dot8<BF>(gst.v[i], ost.v[i]));
            const int row = (int)threadIdx.x / G::CPR + i * (G::NT / G::CPR);
            if (row < G::ZROW && threadIdx.x % G::CPR == 0) lds_stat[row].y = d;
        }
        if (threadIdx.x < G::ZROW) lds_stat[threadIdx.x].x = lse_st * kLog2e;
        __syncthreads();

        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        OTile nxt = cur;
        if (more) {
            nxt = otile_of(tn, ts.tiles_r, ts.tiles_c, s);
            prefetch_qk(nxt);
        }

        // (Passing the lane numbers through an empty asm here, so that the LDS addresses of the
        // unrolled bodies are formed afresh per tile instead of being held in registers across
        // tiles, saves 7 of the 24 spilled registers at kernel_size 7 and costs 6-25% of the time:
        // B8 N2 112x112 56.6 -> 70.6 us.  The compiler's own choice stays.)
        const int n = n_lane, g = g_lane;
        const int br = block_r(cur), bc = block_c(cur);
        // this lane's pixel, as a query and as a key; written by this tile unless it lies in
        // the last 8 rows / columns and this is not the last tile of the axis
        const int wy0 = cur.r0 + (wave >> 1) * 4, wx0 = cur.c0 + (wave & 1) * 4;
        const int py = wy0 + (n >> 2), px = wx0 + (n & 3);
        const bool live = (cur.last_r || py < s.H - 8) && (cur.last_c || px < s.W - 8);
        const int prow = (py - br) * G::HC + (px - bc);
        const int64_t goff = a.grad_at(cur.bb, cur.nn, py, px);
        {
            // ---- dQ: the wave's keys are the (4+k-1)^2 pixels from the window start of its
            // first query row / column on (moved back where that would leave the block)
            const int sy0 = min(win_start(wy0, s.H, KS), br + 4), sx0 = min(win_start(wx0, s.W, KS), bc + 4);
            const int orow = sy0 - br, ocol = sx0 - bc;
            const int dr = win_start(py, s.H, KS) - sy0, dc = win_start(px, s.W, KS) - sx0;
            auto trow = [&](int tile, int x) __attribute__((always_inline)) {
                return G::token_row(tile, x, orow, ocol);
            };
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
            s16x8 dsb[G::KSTEPS];
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
                    const bool ok = G::template tok_in<KS>(mt, g * 4 + i, dr, dc);
                    const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - mine.x : -INFINITY);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - mine.y));
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
            store_token<BF, D>(static_cast<short *>(a.dq) + goff, g, dq, s.scale, live);
        }
        {
            // ---- dK, dV: this lane's key is column n of every product
            s16x8 kreg[G::DS], vreg[G::DS];
            {
                const typename G::ARow kp = G::a_row(lds_k, prow, g), vp = G::a_row(lds_v, prow, g);
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    kreg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(kp, ds));
                    vreg[ds] = *reinterpret_cast<const s16x8 *>(G::a_at(vp, ds));
                }
            }
            f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) {
                dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
                dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
            const int tr = cur.r0 >> 3, tc = cur.c0 >> 3;
            const bool inner = (cur.r0 & 7) == 0 && (cur.c0 & 7) == 0 && tr >= ts.ir0 &&
                               tr < ts.ir0 + ts.ni_r && tc >= ts.ic0 && tc < ts.ic0 + ts.ni_c;
            if (inner) {
                // No key or query of the tile is within reach of a border: every window is
                // centred, the queries of the wave's keys are the (4+k-1)^2 pixels around
                // them at a fixed place in the block, and the mask depends on the lane only.
                const int orow = (wave >> 1) * 4, ocol = (wave & 1) * 4;
                auto row_of = [&](int tile, int x) __attribute__((always_inline)) {
                    return G::token_row(tile, x, orow, ocol);
                };
#pragma unroll
                for (int ks = 0; ks < G::KSTEPS; ks++) {
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
                            const float2 st = lds_stat[row_of(mt, g * 4 + i)];
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
            } else {
                // Beside a border the queries that attend to the wave's 4x4 keys span up to
                // 4 + k - 1 + k/2 rows and columns: their rectangle inside the block, numbered
                // row-major and walked 32 at a time, each query masked by its own window.
                const int ra = max(inv_lo(wy0, KS), br);
                const int rb = min(min(inv_hi(wy0 + 3, s.H, KS), br + G::HR), s.H);
                const int cc = max(inv_lo(wx0, KS), bc);
                const int cd = min(min(inv_hi(wx0 + 3, s.W, KS), bc + G::HC), s.W);
                const int wcols = cd - cc;
                const int nq = (rb - ra) * wcols;
                // qi * magic >> 16 == qi / wcols for qi < 2048, wcols <= 32
                const int magic = (65536 + wcols - 1) / wcols;
                auto row_of = [&](int qi) __attribute__((always_inline)) {
                    const int dvd = (qi * magic) >> 16;
                    const int row = (ra + dvd - br) * G::HC + (cc + qi - dvd * wcols - bc);
                    return qi < nq ? row : (int)G::ZROW;
                };
#pragma unroll 1
                for (int q0 = 0; q0 < nq; q0 += 32) {
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
                            const int dvd = (qi * magic) >> 16;
                            const int er = ra + dvd, ec = cc + qi - dvd * wcols;
                            const float2 st = lds_stat[row_of(qi)];
                            const bool ok = (qi < nq) &
                                            ((unsigned)(py - win_start(er, s.H, KS)) < (unsigned)KS) &
                                            ((unsigned)(px - win_start(ec, s.W, KS)) < (unsigned)KS);
                            const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
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
                        dv[mt] = mfma16<BF>(cat(lds_read_tr(G::t_at(gt[0], mt)), lds_read_tr(G::t_at(gt[1], mt))),
                                            pb, dv[mt]);
                        dk[mt] = mfma16<BF>(cat(lds_read_tr(G::t_at(qt[0], mt)), lds_read_tr(G::t_at(qt[1], mt))),
                                            dsb, dk[mt]);
                    }
                }
            }
            store_token<BF, D>(static_cast<short *>(a.dk) + goff, g, dk, s.scale, live);
            store_token<BF, D>(static_cast<short *>(a.dv) + goff, g, dv, 1.f, live);
        }
        if (more) prefetch_vgo(nxt);

        if (!more) break;
        __syncthreads();  // every wave is done with this tile's LDS
        cur = nxt;
        sc.t = tn;
    }
}

template <bool BF, int D, int KS>
int onepass_launch(const BwdArgs &a, const TileSet &ts, int64_t ntiles, hipStream_t st) {
    if constexpr (OGeo<D, KS>::BUILT) {
        const int grid = persistent_grid<bwd_onepass_mfma<BF, D, KS>>(ntiles);
        ProfScope prof(ENATTEN_KERNEL_BWD_FUSED, "bwd_onepass_mfma", st);
        hipLaunchKernelGGL((bwd_onepass_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, ts, (int)ntiles);
        return ENATTEN_OK;
    } else {
        return ENATTEN_EUNSUPPORTED;
    }
}

}  // namespace

// Built for head_dim 32 with kernel_size 3, 5, 7 and head_dim 64 with kernel_size 3, on
// images with sides of at least 8.
bool onepass_bwd_supported(const BwdArgs &a) {
    const int D = a.s.D, ks = a.s.kh;
    const bool built = (D == 32 && (ks == 3 || ks == 5 || ks == 7)) || (D == 64 && ks == 3);
    return built && a.s.kw == ks && a.s.H >= 8 && a.s.W >= 8;
}

int launch_bwd_onepass(const BwdArgs &a, bool bf16, const TileSet &ts, int64_t ntiles, hipStream_t st) {
#define ENATTEN_ONEPASS(DD, KK)                                              \
    if (a.s.D == DD && a.s.kh == KK)                                         \
        return bf16 ? onepass_launch<true, DD, KK>(a, ts, ntiles, st)        \
                    : onepass_launch<false, DD, KK>(a, ts, ntiles, st);
    ENATTEN_ONEPASS(32, 3)
    ENATTEN_ONEPASS(32, 5)
    ENATTEN_ONEPASS(32, 7)
    ENATTEN_ONEPASS(64, 3)
#undef ENATTEN_ONEPASS
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace enatten
