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
// Forward follows e_natten/triton.py:242-302 per query (window start, mask,
// softmax, P.V); the log-sum-exp is kept for the backward.

#include <math.h>

#include "na2d_common.h"

namespace enatten {
namespace {

typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <bool BF>
__device__ inline f32x4 mfma16(s16x8 a, s16x8 b, f32x4 c) {
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <bool BF>
__device__ inline short cvt16(float x) {
    if constexpr (BF) return __builtin_bit_cast(short, (__bf16)x);
    else return __builtin_bit_cast(short, (_Float16)x);
}

template <bool BF>
__device__ inline float cvt32(short x) {
    if constexpr (BF) return __uint_as_float(((uint32_t)(uint16_t)x) << 16);
    else return (float)__builtin_bit_cast(_Float16, x);
}

// 4 tokens x 16 channels out of channel-major LDS, transposed: lane i of each
// 16-lane group receives, for the channel the caller assigned to it, the values
// of the 4 tokens addressed by lanes {i/4, 4+i/4, 8+i/4, 12+i/4}.
__device__ inline s16x4 lds_read_tr(const short *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3))) *)(p));
}

__device__ inline s16x8 cat(s16x4 lo, s16x4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// max / sum over the four lanes that share a query column (l, l^16, l^32, l^48)
__device__ inline float col_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16, 64));
    return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ inline float col_sum(float x) {
    x += __shfl_xor(x, 16, 64);
    return x + __shfl_xor(x, 32, 64);
}

template <int D, int KS>
struct Geo {
    static constexpr int TH = 8, TW = 8;          // pixels per workgroup
    static constexpr int HR = TH + KS - 1;        // halo of the workgroup tile
    static constexpr int HC = TW + KS - 1;
    static constexpr int SW = 4 + KS - 1;         // halo side of one wave's 4x4 block
    static constexpr int NK = SW * SW;            // halo tokens per wave
    static constexpr int NKP = (NK + 31) / 32 * 32;
    static constexpr int MT = NKP / 16;           // 16-token MFMA row tiles
    static constexpr int KSTEPS = NKP / 32;       // reduction steps of the second product
    static constexpr int PITCH = D + 8;           // LDS row pitch in elements (16 B pad)
    static constexpr int ROWS = HR * HC + 1;      // + one all-zero row for padding tokens
    static constexpr int ZROW = HR * HC;
    static constexpr int CPR = D / 8;             // 16-byte chunks per row
    static constexpr int DS = D / 32;             // reduction steps over channels
    static constexpr int DT = D / 16;             // 16-channel MFMA row tiles of the output
    static constexpr size_t LDS_BYTES =
        (size_t)2 * ROWS * PITCH * sizeof(short) + ROWS * 2 * sizeof(float);
};

// XCD-aware block order: hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs, each with its own L2.  Give every XCD one contiguous run of tiles
// so the halos shared by neighbouring tiles meet in the same L2.
__device__ inline int logical_block(int nblocks) {
    const int per_xcd = gridDim.x >> 3;
    const int id = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    return id < nblocks ? id : -1;
}

// Copy the halo [hr0, hr0+HR) x [hc0, hc0+HC) of one image into LDS, channel-
// major with padded pitch; positions outside the image and the spare row are
// zero so that masked tokens contribute exact zeros to the second product.
template <int D, int KS>
__device__ inline void stage_halo(short *lds, const short *img, int64_t sh, int64_t sw, int hr0,
                                  int hc0, int H, int W) {
    using G = Geo<D, KS>;
    constexpr int NCH = G::HR * G::HC * G::CPR;
    for (int id = threadIdx.x; id < NCH; id += 256) {
        const int row = id / G::CPR, ch = id % G::CPR;
        const int r = hr0 + row / G::HC, c = hc0 + row % G::HC;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (r < H && c < W) v = *reinterpret_cast<const uint4 *>(img + r * sh + c * sw + ch * 8);
        *reinterpret_cast<uint4 *>(lds + row * G::PITCH + ch * 8) = v;
    }
    if (threadIdx.x < G::CPR)
        *reinterpret_cast<uint4 *>(lds + G::ZROW * G::PITCH + threadIdx.x * 8) =
            make_uint4(0, 0, 0, 0);
}

// ------------------------------------------------------------------ forward
template <bool BF, int D, int KS>
__global__ __launch_bounds__(256) void fwd_mfma(FwdArgs a, int tiles_r, int tiles_c,
                                                int nblocks) {
    using G = Geo<D, KS>;
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];

    const Shape &s = a.s;
    int t = logical_block(nblocks);
    if (t < 0) return;
    const int tc = t % tiles_c; t /= tiles_c;
    const int tr = t % tiles_r;
    const int slab = t / tiles_r;
    const int bb = slab / s.N, nn = slab % s.N;
    const int r0 = tr * G::TH, c0 = tc * G::TW;
    const int hr0 = win_start(r0, s.H, KS), hc0 = win_start(c0, s.W, KS);

    const short *kimg = static_cast<const short *>(a.k.ptr) + bb * a.k.sb + nn * a.k.sn;
    const short *vimg = static_cast<const short *>(a.v.ptr) + bb * a.v.sb + nn * a.v.sn;
    stage_halo<D, KS>(lds_k, kimg, a.k.sh, a.k.sw, hr0, hc0, s.H, s.W);
    stage_halo<D, KS>(lds_v, vimg, a.v.sh, a.v.sw, hr0, hc0, s.H, s.W);
    __syncthreads();

    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const int wr0 = r0 + (wave >> 1) * 4, wc0 = c0 + (wave & 1) * 4;
    if (wr0 >= s.H || wc0 >= s.W) return;  // block of 16 queries entirely outside
    const bool live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
    const int qr = min(wr0 + (n >> 2), s.H - 1), qc = min(wc0 + (n & 3), s.W - 1);
    // origin of the wave's halo inside the image and inside the staged halo
    const int sr0 = win_start(wr0, s.H, KS), sc0 = win_start(wc0, s.W, KS);
    const int orow = sr0 - hr0, ocol = sc0 - hc0;
    // this lane's query window, relative to the wave's halo
    const int dr = win_start(qr, s.H, KS) - sr0, dc = win_start(qc, s.W, KS) - sc0;

    // B operand of the first product: this lane's query, channels s*32 + g*8 ..
    const short *qp = static_cast<const short *>(a.q.ptr) + bb * a.q.sb + nn * a.q.sn +
                      qr * a.q.sh + qc * a.q.sw + g * 8;
    s16x8 qreg[G::DS];
#pragma unroll
    for (int ds = 0; ds < G::DS; ds++) qreg[ds] = *reinterpret_cast<const s16x8 *>(qp + ds * 32);

    // logits^T [halo token][query], masked, in units of log2
    const float sc2 = s.scale * kLog2e;
    f32x4 acc[G::MT];
    float mx = -INFINITY;
#pragma unroll
    for (int mt = 0; mt < G::MT; mt++) {
        const int kk = mt * 16 + n;
        const int row = kk < G::NK ? (orow + kk / G::SW) * G::HC + ocol + kk % G::SW : G::ZROW;
        const short *kp = lds_k + row * G::PITCH + g * 8;
        f32x4 c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++)
            c = mfma16<BF>(*reinterpret_cast<const s16x8 *>(kp + ds * 32), qreg[ds], c);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int tk = mt * 16 + g * 4 + i;  // halo token of accumulator row g*4+i
            const int kr = tk / G::SW, kc = tk % G::SW;
            const bool ok = tk < G::NK && (unsigned)(kr - dr) < (unsigned)KS &&
                            (unsigned)(kc - dc) < (unsigned)KS;
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
        const short *vp[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int tk = ks * 32 + h * 16 + g * 4 + (n >> 2);
            const int row = tk < G::NK ? (orow + tk / G::SW) * G::HC + ocol + tk % G::SW : G::ZROW;
            vp[h] = lds_v + row * G::PITCH + (n & 3) * (D / 4);
        }
#pragma unroll
        for (int mt = 0; mt < G::DT; mt++)
            o[mt] = mfma16<BF>(cat(lds_read_tr(vp[0] + mt * 4), lds_read_tr(vp[1] + mt * 4)),
                               pb[ks], o[mt]);
    }

    if (!live) return;
    const float inv = 1.f / sum;
    const int64_t tok = (((int64_t)bb * s.N + nn) * s.H + qr) * s.W + qc;
    short *op = static_cast<short *>(a.o) + tok * D + g * (D / 4);
#pragma unroll
    for (int j = 0; j < G::DT / 2; j++) {
        s16x8 w;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = cvt16<BF>(o[2 * j][i] * inv);
            w[4 + i] = cvt16<BF>(o[2 * j + 1][i] * inv);
        }
        *reinterpret_cast<s16x8 *>(op + j * 8) = w;
    }
    if (a.lse && g == 0) a.lse[tok] = (mx + __builtin_amdgcn_logf(sum)) * kLn2;
}

// ------------------------------------------------------------------ dQ
// Query-centric like the forward: recompute P from the saved log-sum-exp, form
// dP^T = V dO^T on the same halo, dS = P * (dP - delta) with delta = dO . O, and
// dQ^T = K^T dS^T with K read back from LDS transposed.  Also writes delta for the
// dK/dV pass.  Per-query math: e_natten/triton.py:383-398.
template <bool BF, int D, int KS>
__global__ __launch_bounds__(256) void bwd_dq_mfma(BwdArgs a, int tiles_r, int tiles_c,
                                                   int nblocks) {
    using G = Geo<D, KS>;
    __shared__ __attribute__((aligned(16))) short lds_k[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_v[G::ROWS * G::PITCH];

    const Shape &s = a.s;
    int t = logical_block(nblocks);
    if (t < 0) return;
    const int tc = t % tiles_c; t /= tiles_c;
    const int tr = t % tiles_r;
    const int slab = t / tiles_r;
    const int bb = slab / s.N, nn = slab % s.N;
    const int r0 = tr * G::TH, c0 = tc * G::TW;
    const int hr0 = win_start(r0, s.H, KS), hc0 = win_start(c0, s.W, KS);

    const short *kimg = static_cast<const short *>(a.k.ptr) + bb * a.k.sb + nn * a.k.sn;
    const short *vimg = static_cast<const short *>(a.v.ptr) + bb * a.v.sb + nn * a.v.sn;
    stage_halo<D, KS>(lds_k, kimg, a.k.sh, a.k.sw, hr0, hc0, s.H, s.W);
    stage_halo<D, KS>(lds_v, vimg, a.v.sh, a.v.sw, hr0, hc0, s.H, s.W);
    __syncthreads();

    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const int wr0 = r0 + (wave >> 1) * 4, wc0 = c0 + (wave & 1) * 4;
    if (wr0 >= s.H || wc0 >= s.W) return;
    const bool live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
    const int qr = min(wr0 + (n >> 2), s.H - 1), qc = min(wc0 + (n & 3), s.W - 1);
    const int sr0 = win_start(wr0, s.H, KS), sc0 = win_start(wc0, s.W, KS);
    const int orow = sr0 - hr0, ocol = sc0 - hc0;
    const int dr = win_start(qr, s.H, KS) - sr0, dc = win_start(qc, s.W, KS) - sc0;

    const int64_t tok = (((int64_t)bb * s.N + nn) * s.H + qr) * s.W + qc;
    const short *qp = static_cast<const short *>(a.q.ptr) + bb * a.q.sb + nn * a.q.sn +
                      qr * a.q.sh + qc * a.q.sw + g * 8;
    const short *gp = static_cast<const short *>(a.d_o) + tok * D + g * 8;
    const short *op = static_cast<const short *>(a.o) + tok * D + g * 8;
    s16x8 qreg[G::DS], greg[G::DS];
    float dpart = 0.f;
#pragma unroll
    for (int ds = 0; ds < G::DS; ds++) {
        qreg[ds] = *reinterpret_cast<const s16x8 *>(qp + ds * 32);
        greg[ds] = *reinterpret_cast<const s16x8 *>(gp + ds * 32);
        const s16x8 orow8 = *reinterpret_cast<const s16x8 *>(op + ds * 32);
#pragma unroll
        for (int e = 0; e < 8; e++) dpart = fmaf(cvt32<BF>(greg[ds][e]), cvt32<BF>(orow8[e]), dpart);
    }
    const float delta = col_sum(dpart);
    const float lse2 = a.lse[tok] * kLog2e;
    const float sc2 = s.scale * kLog2e;

    s16x8 dsb[G::KSTEPS];
#pragma unroll
    for (int mt = 0; mt < G::MT; mt++) {
        const int kk = mt * 16 + n;
        const int row = kk < G::NK ? (orow + kk / G::SW) * G::HC + ocol + kk % G::SW : G::ZROW;
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
            const int tk = mt * 16 + g * 4 + i;
            const int kr = tk / G::SW, kc = tk % G::SW;
            const bool ok = tk < G::NK && (unsigned)(kr - dr) < (unsigned)KS &&
                            (unsigned)(kc - dc) < (unsigned)KS;
            const float p = ok ? __builtin_amdgcn_exp2f(cs[i] * sc2 - lse2) : 0.f;
            dsb[mt >> 1][(mt & 1) * 4 + i] = cvt16<BF>(p * (cp[i] - delta));
        }
    }

    f32x4 dq[G::DT];
#pragma unroll
    for (int mt = 0; mt < G::DT; mt++) dq[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < G::KSTEPS; ks++) {
        const short *kp[2];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int tk = ks * 32 + h * 16 + g * 4 + (n >> 2);
            const int row = tk < G::NK ? (orow + tk / G::SW) * G::HC + ocol + tk % G::SW : G::ZROW;
            kp[h] = lds_k + row * G::PITCH + (n & 3) * (D / 4);
        }
#pragma unroll
        for (int mt = 0; mt < G::DT; mt++)
            dq[mt] = mfma16<BF>(cat(lds_read_tr(kp[0] + mt * 4), lds_read_tr(kp[1] + mt * 4)),
                                dsb[ks], dq[mt]);
    }

    if (!live) return;
    short *dqp = static_cast<short *>(a.dq) + tok * D + g * (D / 4);
#pragma unroll
    for (int j = 0; j < G::DT / 2; j++) {
        s16x8 w;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = cvt16<BF>(dq[2 * j][i] * s.scale);
            w[4 + i] = cvt16<BF>(dq[2 * j + 1][i] * s.scale);
        }
        *reinterpret_cast<s16x8 *>(dqp + j * 8) = w;
    }
    if (g == 0) a.delta[tok] = delta;
}

// ------------------------------------------------------------------ dK, dV
// Key-centric: the workgroup owns an 8x8 tile of keys and stages Q, dO, the
// log-sum-exp and delta of the queries that attend to them, i.e. the union of the
// keys' inverse neighbourhoods (e_natten/pytorch.py:13-23, :261-270).  That union
// is (8+k-1)^2 queries in the interior and larger beside an image edge (the
// clamped windows of the k//2 border queries all reach k pixels in), so it is
// walked in blocks of at most (8+k-1)^2 queries, restaging LDS per block.  Each
// wave owns 4x4 keys (MFMA columns) and walks the queries of the block that can
// attend to them, 32 at a time:
//   S = Q K^T, dP = dO V^T           (query rows from LDS, key columns in registers)
//   P = exp(S - lse), dS = P (dP - delta), masked to the query's own window
//   dV^T += dO^T P, dK^T += Q^T dS    (dO, Q read back from LDS transposed)
template <bool BF, int D, int KS>
__global__ __launch_bounds__(256) void bwd_dkdv_mfma(BwdArgs a, int tiles_r, int tiles_c,
                                                     int nblocks) {
    using G = Geo<D, KS>;
    __shared__ __attribute__((aligned(16))) short lds_q[G::ROWS * G::PITCH];
    __shared__ __attribute__((aligned(16))) short lds_g[G::ROWS * G::PITCH];
    __shared__ float2 lds_stat[G::ROWS];  // (lse * log2e, delta) per staged query

    const Shape &s = a.s;
    int t = logical_block(nblocks);
    if (t < 0) return;
    const int tc = t % tiles_c; t /= tiles_c;
    const int tr = t % tiles_r;
    const int slab = t / tiles_r;
    const int bb = slab / s.N, nn = slab % s.N;
    const int r0 = tr * G::TH, c0 = tc * G::TW;
    // queries that attend to any key of the tile
    const int qa = inv_lo(r0, KS), qb = inv_hi(min(r0 + G::TH, s.H) - 1, s.H, KS);
    const int ca = inv_lo(c0, KS), cb = inv_hi(min(c0 + G::TW, s.W) - 1, s.W, KS);

    const int wave = threadIdx.x >> 6, l = threadIdx.x & 63, n = l & 15, g = l >> 4;
    const int wr0 = r0 + (wave >> 1) * 4, wc0 = c0 + (wave & 1) * 4;
    const bool wave_on = wr0 < s.H && wc0 < s.W;
    const bool live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
    const int kr = min(wr0 + (n >> 2), s.H - 1), kc = min(wc0 + (n & 3), s.W - 1);
    // queries that attend to any key of this wave's 4x4 block
    const int wqa = wave_on ? inv_lo(wr0, KS) : 0;
    const int wqb = wave_on ? inv_hi(min(wr0 + 4, s.H) - 1, s.H, KS) : 0;
    const int wca = wave_on ? inv_lo(wc0, KS) : 0;
    const int wcb = wave_on ? inv_hi(min(wc0 + 4, s.W) - 1, s.W, KS) : 0;

    const short *qimg = static_cast<const short *>(a.q.ptr) + bb * a.q.sb + nn * a.q.sn;
    const int64_t img_tok = ((int64_t)bb * s.N + nn) * s.H * (int64_t)s.W;
    const short *gimg = static_cast<const short *>(a.d_o) + img_tok * D;

    // B operands: this lane's key, channels ds*32 + g*8 ..
    s16x8 kreg[G::DS], vreg[G::DS];
    {
        const short *kp = static_cast<const short *>(a.k.ptr) + bb * a.k.sb + nn * a.k.sn +
                          kr * a.k.sh + kc * a.k.sw + g * 8;
        const short *vp = static_cast<const short *>(a.v.ptr) + bb * a.v.sb + nn * a.v.sn +
                          kr * a.v.sh + kc * a.v.sw + g * 8;
#pragma unroll
        for (int ds = 0; ds < G::DS; ds++) {
            kreg[ds] = *reinterpret_cast<const s16x8 *>(kp + ds * 32);
            vreg[ds] = *reinterpret_cast<const s16x8 *>(vp + ds * 32);
        }
    }
    const float sc2 = s.scale * kLog2e;
    f32x4 dk[G::DT], dv[G::DT];
#pragma unroll
    for (int mt = 0; mt < G::DT; mt++) {
        dk[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        dv[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    for (int br = qa; br < qb; br += G::HR) {
        for (int bc = ca; bc < cb; bc += G::HC) {
            if (br != qa || bc != ca) __syncthreads();  // previous block fully consumed
            stage_halo<D, KS>(lds_q, qimg, a.q.sh, a.q.sw, br, bc, qb, cb);
            stage_halo<D, KS>(lds_g, gimg, (int64_t)s.W * D, D, br, bc, qb, cb);
            for (int id = threadIdx.x; id < G::ROWS; id += 256) {
                const int r = br + id / G::HC, c = bc + id % G::HC;
                float2 st = make_float2(0.f, 0.f);
                if (id < G::ZROW && r < qb && c < cb) {
                    const int64_t qt = img_tok + (int64_t)r * s.W + c;
                    st = make_float2(a.lse[qt] * kLog2e, a.delta[qt]);
                }
                lds_stat[id] = st;
            }
            __syncthreads();

            // this wave's queries inside the staged block
            const int ra = max(wqa, br), rb = min(wqb, br + G::HR);
            const int cc = max(wca, bc), cd = min(wcb, bc + G::HC);
            const int wcols = cd - cc;
            const int nq = (rb > ra && cd > cc) ? (rb - ra) * wcols : 0;
            const int magic = wcols > 0 ? (65536 + wcols - 1) / wcols : 0;
            // staged row of the wave's query number qi (row-major over its rectangle)
            auto row_of = [&](int qi, int &r, int &c) {
                const int dvd = (qi * magic) >> 16;
                r = ra + dvd;
                c = cc + qi - dvd * wcols;
                return qi < nq ? (r - br) * G::HC + (c - bc) : (int)G::ZROW;
            };
            for (int q0 = 0; q0 < nq; q0 += 32) {
                s16x8 pb, dsb;
#pragma unroll
                for (int m2 = 0; m2 < 2; m2++) {
                    int rr, rc;
                    const int row = row_of(q0 + m2 * 16 + n, rr, rc);
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
                        const int qi = q0 + m2 * 16 + g * 4 + i;
                        int er, ec;
                        const int erow = row_of(qi, er, ec);
                        const float2 st = lds_stat[erow];
                        const bool ok = qi < nq &&
                                        (unsigned)(kr - win_start(er, s.H, KS)) < (unsigned)KS &&
                                        (unsigned)(kc - win_start(ec, s.W, KS)) < (unsigned)KS;
                        const float p = ok ? __builtin_amdgcn_exp2f(cs[i] * sc2 - st.x) : 0.f;
                        pb[m2 * 4 + i] = cvt16<BF>(p);
                        dsb[m2 * 4 + i] = cvt16<BF>(p * (cp[i] - st.y));
                    }
                }
                const short *qt[2], *gt[2];
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    int rr, rc;
                    const int row = row_of(q0 + h * 16 + g * 4 + (n >> 2), rr, rc);
                    qt[h] = lds_q + row * G::PITCH + (n & 3) * (D / 4);
                    gt[h] = lds_g + row * G::PITCH + (n & 3) * (D / 4);
                }
#pragma unroll
                for (int mt = 0; mt < G::DT; mt++) {
                    dv[mt] = mfma16<BF>(
                        cat(lds_read_tr(gt[0] + mt * 4), lds_read_tr(gt[1] + mt * 4)), pb, dv[mt]);
                    dk[mt] = mfma16<BF>(
                        cat(lds_read_tr(qt[0] + mt * 4), lds_read_tr(qt[1] + mt * 4)), dsb, dk[mt]);
                }
            }
        }
    }

    if (!live) return;
    const int64_t tok = img_tok + (int64_t)kr * s.W + kc;
    short *dkp = static_cast<short *>(a.dk) + tok * D + g * (D / 4);
    short *dvp = static_cast<short *>(a.dv) + tok * D + g * (D / 4);
#pragma unroll
    for (int j = 0; j < G::DT / 2; j++) {
        s16x8 wk, wv;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            wk[i] = cvt16<BF>(dk[2 * j][i] * s.scale);
            wk[4 + i] = cvt16<BF>(dk[2 * j + 1][i] * s.scale);
            wv[i] = cvt16<BF>(dv[2 * j][i]);
            wv[4 + i] = cvt16<BF>(dv[2 * j + 1][i]);
        }
        *reinterpret_cast<s16x8 *>(dkp + j * 8) = wk;
        *reinterpret_cast<s16x8 *>(dvp + j * 8) = wv;
    }
}

// ------------------------------------------------------------------ dispatch
template <int D, int KS>
constexpr bool fits() {
    return Geo<D, KS>::LDS_BYTES <= 160 * 1024;
}

int check_launch(const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        set_error("%s: launch failed: %s", what, hipGetErrorString(e));
        return ENATTEN_ELAUNCH;
    }
    return ENATTEN_OK;
}

bool layout_ok(const View &v) {
    return reinterpret_cast<uintptr_t>(v.ptr) % 16 == 0 && v.sb % 8 == 0 && v.sn % 8 == 0 &&
           v.sh % 8 == 0 && v.sw % 8 == 0;
}

template <bool BF, int D, int KS>
int fwd_launch(const FwdArgs &a, hipStream_t st) {
    if constexpr (fits<D, KS>()) {
        using G = Geo<D, KS>;
        const int tiles_r = (a.s.H + G::TH - 1) / G::TH, tiles_c = (a.s.W + G::TW - 1) / G::TW;
        const int64_t nb = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
        const int grid = (int)((nb + 7) / 8 * 8);
        {
            ProfScope prof(ENATTEN_KERNEL_FWD, "fwd_mfma", st);
            hipLaunchKernelGGL((fwd_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, tiles_r,
                               tiles_c, (int)nb);
        }
        return check_launch("enatten2d_fwd");
    } else {
        set_error("no matrix-core kernel for head_dim %d, kernel_size %d", D, KS);
        return ENATTEN_EUNSUPPORTED;
    }
}

template <bool BF, int D, int KS>
int bwd_launch(const BwdArgs &a, hipStream_t st) {
    if constexpr (fits<D, KS>()) {
        using G = Geo<D, KS>;
        const int tiles_r = (a.s.H + G::TH - 1) / G::TH, tiles_c = (a.s.W + G::TW - 1) / G::TW;
        const int64_t nb = (int64_t)a.s.B * a.s.N * tiles_r * tiles_c;
        const int grid = (int)((nb + 7) / 8 * 8);
        {
            ProfScope prof(ENATTEN_KERNEL_BWD_DQ, "bwd_dq_mfma", st);
            hipLaunchKernelGGL((bwd_dq_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, tiles_r,
                               tiles_c, (int)nb);
        }
        {
            ProfScope prof(ENATTEN_KERNEL_BWD_DKDV, "bwd_dkdv_mfma", st);
            hipLaunchKernelGGL((bwd_dkdv_mfma<BF, D, KS>), dim3(grid), dim3(256), 0, st, a, tiles_r,
                               tiles_c, (int)nb);
        }
        return check_launch("enatten2d_bwd");
    } else {
        set_error("no matrix-core kernel for head_dim %d, kernel_size %d", D, KS);
        return ENATTEN_EUNSUPPORTED;
    }
}

#define ENATTEN_BY_KS(FN, BF, D, ARGS, ST)                       \
    switch ((ARGS).s.kh) {                                       \
        case 3: return FN<BF, D, 3>(ARGS, ST);                   \
        case 5: return FN<BF, D, 5>(ARGS, ST);                   \
        case 7: return FN<BF, D, 7>(ARGS, ST);                   \
        case 9: return FN<BF, D, 9>(ARGS, ST);                   \
        case 11: return FN<BF, D, 11>(ARGS, ST);                 \
        case 13: return FN<BF, D, 13>(ARGS, ST);                 \
    }

#define ENATTEN_BY_D(FN, BF, ARGS, ST)                           \
    switch ((ARGS).s.D) {                                        \
        case 32: ENATTEN_BY_KS(FN, BF, 32, ARGS, ST) break;      \
        case 64: ENATTEN_BY_KS(FN, BF, 64, ARGS, ST) break;      \
        case 128: ENATTEN_BY_KS(FN, BF, 128, ARGS, ST) break;    \
    }

bool fits_rt(int D, int ks) {
    const int rows = (8 + ks - 1) * (8 + ks - 1) + 1;
    return (size_t)2 * rows * (D + 8) * 2 + (size_t)rows * 8 <= 160 * 1024;
}

}  // namespace

bool mfma_supported(int D, int ks, int dtype) {
    if (dtype != ENATTEN_BF16 && dtype != ENATTEN_F16) return false;
    if (D != 32 && D != 64 && D != 128) return false;
    if (ks < 3 || ks > 13 || ks % 2 == 0) return false;
    return fits_rt(D, ks);
}

int launch_fwd_mfma(const FwdArgs &a, int dtype, hipStream_t st) {
    if (!layout_ok(a.q) || !layout_ok(a.k) || !layout_ok(a.v) ||
        reinterpret_cast<uintptr_t>(a.o) % 16 != 0)
        return launch_fwd_simt(a, dtype, st);  // 16-byte loads need aligned rows
    if (dtype == ENATTEN_BF16) {
        ENATTEN_BY_D(fwd_launch, true, a, st)
    } else {
        ENATTEN_BY_D(fwd_launch, false, a, st)
    }
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

int launch_bwd_mfma(const BwdArgs &a, int dtype, hipStream_t st) {
    auto al = [](const void *p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
    if (!layout_ok(a.q) || !layout_ok(a.k) || !layout_ok(a.v) || !al(a.o) || !al(a.d_o) ||
        !al(a.dq) || !al(a.dk) || !al(a.dv))
        return launch_bwd_simt(a, dtype, st);
    if (dtype == ENATTEN_BF16) {
        ENATTEN_BY_D(bwd_launch, true, a, st)
    } else {
        ENATTEN_BY_D(bwd_launch, false, a, st)
    }
    set_error("no matrix-core kernel for head_dim %d, kernel_size %d", a.s.D, a.s.kh);
    return ENATTEN_EUNSUPPORTED;
}

}  // namespace enatten
