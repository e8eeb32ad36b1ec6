// Fused backward of 2D neighborhood attention on the matrix cores of gfx950:
// dQ, dK and dV of an 8x8 tile of pixels from ONE staging of the tile's
// (8+k-1)^2 halo of q, k, v and dO, so that the backward reads each input once
// (the split passes of na2d_mfma.hip read them twice).
//
// A workgroup is eight waves around one copy of the halo in LDS (all four
// tensors, which is why only one workgroup fits a CU):
//   waves 0-3  query side: dQ of their 4x4 queries over the keys of the halo
//              (e_natten/triton.py:383-398 per query);
//   waves 4-7  key side: dK, dV of their 4x4 keys over the queries of the halo
//              (the inverse neighbourhood of e_natten/pytorch.py:13-23, :261-288).
// Both sides recompute P from the saved log-sum-exp.  delta = dO . O of the halo's
// queries is formed while the halo is written to LDS (the forward output is read
// for this and for nothing else).  The MFMA operand layouts, the token numbering
// and the transposing LDS reads are those of na2d_mfma.hip.
//
// The kernel is persistent like the others: the next tile's halo travels from
// HBM into registers while the current tile is computed out of LDS.

#include <type_traits>

#include "na2d_mfma.h"

namespace enatten {
namespace {

template <int D, int KS>
struct FGeo {
    using G = Geo<D, KS>;
    static constexpr int NT = 512;                       // threads per workgroup
    static constexpr int RP = NT / G::CPR;               // halo rows staged per pass
    static constexpr int NL = (G::HR * G::HC + RP - 1) / RP;  // passes (chunks per thread and tensor)
    static constexpr size_t LDS_BYTES =
        (size_t)4 * G::ROWS * G::PITCH * sizeof(short) + (size_t)2 * G::ROWS * sizeof(float);
    static constexpr bool FITS = LDS_BYTES <= 160 * 1024;
};

template <int NL>
struct Chunks {
    u32x4 v[NL];
};

// dO . O over the 8 channels of one 16-byte chunk, in float32 FMAs.  The halves of
// a dword are taken apart with integer operations: a bit_cast of a vector element
// to a 2-vector of 16-bit floats makes this compiler read the chunk's first dword
// four times (seen in the generated code, and in wrong results).
template <bool BF>
__device__ __forceinline__ float half_of(uint32_t w, bool high) {
    const uint32_t h = high ? w >> 16 : w & 0xffffu;
    if constexpr (BF) return __uint_as_float(h << 16);
    else return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
template <bool BF>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b) {
    float even = 0.f, odd = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        even = fmaf(half_of<BF>(a[j], false), half_of<BF>(b[j], false), even);
        odd = fmaf(half_of<BF>(a[j], true), half_of<BF>(b[j], true), odd);
    }
    return even + odd;
}
// sum over aligned groups of LANES (4, 8 or 16) consecutive lanes, in every lane
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
    auto step = [&](auto ctrl) __attribute__((always_inline)) {
        x += __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(x), decltype(ctrl)::value, 0xf, 0xf, true));
    };
    step(std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    step(std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
    if constexpr (LANES >= 8) step(std::integral_constant<int, 0x141>{});   // row_half_mirror
    if constexpr (LANES >= 16) step(std::integral_constant<int, 0x140>{});  // row_mirror
    return x;
}

template <bool BF, int D, int KS>
__global__ __launch_bounds__(512) void bwd_fused_mfma(BwdArgs a, TileSet ts, int ntiles) {
    using G = Geo<D, KS>;
    using F = FGeo<D, KS>;
    __shared__ __attribute__((aligned(16))) short lds_q[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];
    __shared__ float2 lds_stat[G::ROWS];  // (log-sum-exp * log2(e), dO . O) per staged query

    const Shape &s = a.s;
    Sched sc = make_sched(ntiles, blockIdx.x, gridDim.x);
    if (sc.t >= sc.t_end) return;
    const int tid = threadIdx.x;
    if (tid < G::CPR) {
        const u32x4 z = {0u, 0u, 0u, 0u};
        *reinterpret_cast<u32x4 *>(lds_q + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_g + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_k + G::ZROW * G::PITCH + tid * 8) = z;
        *reinterpret_cast<u32x4 *>(lds_v + G::ZROW * G::PITCH + tid * 8) = z;
    }
    if (tid == 0) lds_stat[G::ZROW] = make_float2(0.f, 0.f);

    const int wave = tid >> 6, l = tid & 63, n = l & 15, g = l >> 4;
    const int role = wave >> 2, w = wave & 3;
    const float sc2 = s.scale * kLog2e;
    // origin of the wave's (4+k-1)^2 halo inside the staged block, and the place of
    // this lane's pixel (query or key) in the block
    const int orow = (w >> 1) * 4, ocol = (w & 1) * 4;
    const int prow = (KS / 2 + orow + (n >> 2)) * G::HC + KS / 2 + ocol + (n & 3);
    auto row_of = [&](int tk) __attribute__((always_inline)) {
        return G::token_row(tk, orow, ocol);
    };

    // staging plan: chunk i of this thread is channel chunk tid % CPR of block row
    // tid / CPR + i * RP
    const int ch8 = (tid % G::CPR) * 8;
    const int srow = tid / G::CPR;
    Chunks<F::NL> qst, gst, kst, vst, ost;
    float lse_st = 0.f;
    // q, k, v rows are laid out like dO and O here (stride W*D between rows, D
    // between pixels; checked on the host), so one set of offsets serves all five
    unsigned off[F::NL];
#pragma unroll
    for (int i = 0; i < F::NL; i++) {
        const int row = min(srow + i * F::RP, G::ZROW - 1);  // tail: harmless duplicate
        off[i] = ((unsigned)(row / G::HC) * (unsigned)s.W + (unsigned)(row % G::HC)) * (D * 2u) +
                 (unsigned)ch8 * 2u;
    }
    auto fetch = [&](Chunks<F::NL> &reg, const short *origin) __attribute__((always_inline)) {
        const char *base = reinterpret_cast<const char *>(origin);
#pragma unroll
        for (int i = 0; i < F::NL; i++)
            reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off[i]);
    };
    // The loads of a tile are issued in five parts (one tensor each) spread over
    // the math of the previous tile: a CU only takes so many vector loads at a
    // time, and a wave that waits at the queue with all of them at once does no
    // math meanwhile.
    auto prefetch_part = [&](const Tile &tl, int part) __attribute__((always_inline)) {
        const int64_t img_tok = ((int64_t)tl.bb * s.N + tl.nn) * s.H * (int64_t)s.W;
        const int br = tl.r0 - KS / 2, bc = tl.c0 - KS / 2;
        const int64_t org = ((int64_t)br * s.W + bc) * D;
        if (part == 0) {
            fetch(qst, image<short>(a.q, tl) + org);
            const int id = min(tid, G::ZROW - 1);
            lse_st = a.lse[img_tok + (int64_t)(br + id / G::HC) * s.W + bc + id % G::HC];
        } else if (part == 1) {
            fetch(kst, image<short>(a.k, tl) + org);
        } else if (part == 2) {
            fetch(vst, image<short>(a.v, tl) + org);
        } else if (part == 3) {
            fetch(gst, static_cast<const short *>(a.d_o) + img_tok * D + org);
        } else {
            fetch(ost, static_cast<const short *>(a.o) + img_tok * D + org);
        }
    };
    auto commit = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < F::NL; i++) {
            const int row = srow + i * F::RP;
            const float d = group_sum<G::CPR>(dot8<BF>(gst.v[i], ost.v[i]));
            if (row < G::ZROW) {
                const int e = row * G::PITCH + ch8;
                *reinterpret_cast<u32x4 *>(lds_q + e) = qst.v[i];
                *reinterpret_cast<u32x4 *>(lds_g + e) = gst.v[i];
                *reinterpret_cast<u32x4 *>(lds_k + e) = kst.v[i];
                *reinterpret_cast<u32x4 *>(lds_v + e) = vst.v[i];
                if (ch8 == 0) lds_stat[row].y = d;
            }
        }
        if (tid < G::ZROW) lds_stat[tid].x = lse_st * kLog2e;
    };

    Tile cur = inner_tile(sc.t, ts, s.N);
#pragma unroll
    for (int part = 0; part < 5; part++) prefetch_part(cur, part);
    for (;;) {
        commit();
        __syncthreads();

        const int tn = sc.t + sc.step;
        const bool more = tn < sc.t_end;
        const Tile nxt = more ? inner_tile(tn, ts, s.N) : cur;
        auto issue = [&](int part) __attribute__((always_inline)) {
            __builtin_amdgcn_sched_barrier(0);
            if (more) prefetch_part(nxt, part);
            __builtin_amdgcn_sched_barrier(0);
        };
        const int pr = cur.r0 + orow + (n >> 2), pc = cur.c0 + ocol + (n & 3);
        const int64_t tok = (((int64_t)cur.bb * s.N + cur.nn) * s.H + pr) * s.W + pc;
        if (role == 0) {
            // ---- query side: this lane's query is column n of every product
            s16x8 qreg[G::DS], greg[G::DS];
#pragma unroll
            for (int ds = 0; ds < G::DS; ds++) {
                qreg[ds] = *reinterpret_cast<const s16x8 *>(lds_q + prow * G::PITCH + ds * 32 + g * 8);
                greg[ds] = *reinterpret_cast<const s16x8 *>(lds_g + prow * G::PITCH + ds * 32 + g * 8);
            }
            const float2 mine = lds_stat[prow];
            const float lse2 = mine.x, delta = mine.y;
            s16x8 dsb[G::KSTEPS];
#pragma unroll
            for (int mt = 0; mt < G::MT; mt++) {
                if (mt < 4) issue(mt);
                const int row = row_of(mt * 16 + n);
                const short *kp = lds_k + row * G::PITCH + g * 8;
                const short *vp = lds_v + row * G::PITCH + g * 8;
                f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(kp + ds * 32), qreg[ds], cs);
                    cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(vp + ds * 32), greg[ds], cp);
                }
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int tk = mt * 16 + g * 4 + i;  // key of accumulator row g*4+i
                    const bool ok = tk < G::NK &&
                                    (unsigned)(tk / G::SWC - (n >> 2)) < (unsigned)KS &&
                                    (unsigned)(tk % G::SWC - (n & 3)) < (unsigned)KS;
                    const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - lse2 : -INFINITY);
                    dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - delta));
                }
            }
            issue(4);
            f32x4 dq[G::DT];
#pragma unroll
            for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < G::KSTEPS; ks++) {
                const short *kp[2];
#pragma unroll
                for (int h = 0; h < 2; h++)
                    kp[h] = lds_k + row_of(ks * 32 + h * 16 + g * 4 + (n >> 2)) * G::PITCH +
                            (n & 3) * (D / 4);
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++)
                    dq[mt] = mfma16<BF>(
                        cat(lds_read_tr(kp[0] + mt * 4), lds_read_tr(kp[1] + mt * 4)), dsb[ks],
                        dq[mt]);
            }
            short *dqp = static_cast<short *>(a.dq) + tok * D + g * (D / 4);
#pragma unroll
            for (int j = 0; j < G::DT / 2; j++) {
                s16x8 wq;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    wq[i] = cvt16<BF>(dq[2 * j][i] * s.scale);
                    wq[4 + i] = cvt16<BF>(dq[2 * j + 1][i] * s.scale);
                }
                *reinterpret_cast<s16x8 *>(dqp + j * 8) = wq;
            }
            if (g == 0) a.delta[tok] = delta;  // the passes over the border tiles read it
        } else {
            // ---- key side: this lane's key is column n of every product.  P and dS
            // of all the halo's queries first, then dV and dK one after the other:
            // one accumulator at a time leaves the registers to the next tile's halo.
            s16x8 pb[G::KSTEPS], dsb[G::KSTEPS];
            {
                s16x8 kreg[G::DS], vreg[G::DS];
#pragma unroll
                for (int ds = 0; ds < G::DS; ds++) {
                    kreg[ds] = *reinterpret_cast<const s16x8 *>(lds_k + prow * G::PITCH + ds * 32 + g * 8);
                    vreg[ds] = *reinterpret_cast<const s16x8 *>(lds_v + prow * G::PITCH + ds * 32 + g * 8);
                }
#pragma unroll
                for (int mt = 0; mt < G::MT; mt++) {
                    if (mt < 4) issue(mt);
                    const int row = row_of(mt * 16 + n);
                    const short *qp = lds_q + row * G::PITCH + g * 8;
                    const short *gp = lds_g + row * G::PITCH + g * 8;
                    f32x4 cs = {0.f, 0.f, 0.f, 0.f}, cp = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ds = 0; ds < G::DS; ds++) {
                        cs = mfma16<BF>(*reinterpret_cast<const s16x8 *>(qp + ds * 32), kreg[ds], cs);
                        cp = mfma16<BF>(*reinterpret_cast<const s16x8 *>(gp + ds * 32), vreg[ds], cp);
                    }
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const int tk = mt * 16 + g * 4 + i;  // query of accumulator row g*4+i
                        const float2 st = lds_stat[row_of(tk)];
                        const bool ok = tk < G::NK &&
                                        (unsigned)(tk / G::SWC - (n >> 2)) < (unsigned)KS &&
                                        (unsigned)(tk % G::SWC - (n & 3)) < (unsigned)KS;
                        const float p = __builtin_amdgcn_exp2f(ok ? cs[i] * sc2 - st.x : -INFINITY);
                        pb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p);
                        dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                    }
                }
            }
            auto second = [&](const short *lds_x, const s16x8 (&b)[G::KSTEPS], void *out, float mul)
                              __attribute__((always_inline)) {
                f32x4 acc[G::DT];
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < G::KSTEPS; ks++) {
                    const short *xt[2];
#pragma unroll
                    for (int h = 0; h < 2; h++)
                        xt[h] = lds_x + row_of(ks * 32 + h * 16 + g * 4 + (n >> 2)) * G::PITCH +
                                (n & 3) * (D / 4);
#pragma unroll
                    for (int mt = 0; mt < G::DT; mt++)
                        acc[mt] = mfma16<BF>(
                            cat(lds_read_tr(xt[0] + mt * 4), lds_read_tr(xt[1] + mt * 4)), b[ks],
                            acc[mt]);
                }
                short *op = static_cast<short *>(out) + tok * D + g * (D / 4);
#pragma unroll
                for (int j = 0; j < G::DT / 2; j++) {
                    s16x8 wv;
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        wv[i] = cvt16<BF>(acc[2 * j][i] * mul);
                        wv[4 + i] = cvt16<BF>(acc[2 * j + 1][i] * mul);
                    }
                    *reinterpret_cast<s16x8 *>(op + j * 8) = wv;
                }
            };
            issue(4);
            second(lds_g, pb, a.dv, 1.f);
            second(lds_q, dsb, a.dk, s.scale);
        }
        if (!more) break;
        __syncthreads();  // every wave is done with this tile's LDS
        cur = nxt;
        sc.t = tn;
    }
}

template <bool BF, int D, int KS>
int fused_launch(const BwdArgs &a, const TileSet &ts, int64_t n_inner, hipStream_t st) {
    if constexpr (FGeo<D, KS>::FITS) {
        const int64_t per_xcd = (n_inner + 7) / 8;
        const int grid = (int)(8 * (per_xcd < 32 ? per_xcd : 32));  // one workgroup per CU
        ProfScope prof(ENATTEN_KERNEL_BWD_FUSED, "bwd_fused_mfma", st);
        hipLaunchKernelGGL((bwd_fused_mfma<BF, D, KS>), dim3(grid), dim3(512), 0, st, a, ts,
                           (int)n_inner);
        return ENATTEN_OK;
    } else {
        return ENATTEN_EUNSUPPORTED;
    }
}

}  // namespace

bool fused_bwd_supported(int D, int ks) {
    return D == 128 && ks == 5;
}

// dQ, dK, dV of the inner tiles of `ts` (and delta of their queries, for the
// passes that serve the border tiles).
int launch_bwd_fused_inner(const BwdArgs &a, bool bf16, const TileSet &ts, int64_t n_inner,
                           hipStream_t st) {
    if (a.s.D == 128 && a.s.kh == 5) {
        if (bf16) return fused_launch<true, 128, 5>(a, ts, n_inner, st);
        return fused_launch<false, 128, 5>(a, ts, n_inner, st);
    }
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace enatten
