// Device helpers shared by the matrix-core (MFMA) kernels for 2D neighborhood
// attention on gfx950: operand types, tile geometry, the persistent tile schedule
// and the global -> register -> LDS staging of a tile's halo.
#pragma once

#include <math.h>

#include <type_traits>

#include "na2d_common.h"

namespace enatten {
namespace {

typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));  // 16 bytes in flight
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

template <bool BF>
__device__ __forceinline__ f32x4 mfma16(s16x8 a, s16x8 b, f32x4 c) {
    if constexpr (BF)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                       __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                      __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
}

template <bool BF>
__device__ __forceinline__ short cvt16(float x) {
    if constexpr (BF) return __builtin_bit_cast(short, (__bf16)x);
    else return __builtin_bit_cast(short, (_Float16)x);
}

template <bool BF>
__device__ __forceinline__ float cvt32(short x) {
    if constexpr (BF) return __uint_as_float(((uint32_t)(uint16_t)x) << 16);
    else return (float)__builtin_bit_cast(_Float16, x);
}

// 4 tokens x 16 channels out of channel-major LDS, transposed: lane i of each
// 16-lane group receives, for the channel the caller assigned to it, the values
// of the 4 tokens addressed by lanes {i/4, 4+i/4, 8+i/4, 12+i/4}.
__device__ __forceinline__ s16x4 lds_read_tr(const short *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (s16x4 __attribute__((address_space(3))) *)(p));
}

__device__ __forceinline__ s16x8 cat(s16x4 lo, s16x4 hi) {
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

// max / sum over the four lanes that share a query column (l, l^16, l^32, l^48)
__device__ __forceinline__ float col_max(float x) {
    x = fmaxf(x, __shfl_xor(x, 16, 64));
    return fmaxf(x, __shfl_xor(x, 32, 64));
}
__device__ __forceinline__ float col_sum(float x) {
    x += __shfl_xor(x, 16, 64);
    return x + __shfl_xor(x, 32, 64);
}

// dO . O over the 8 channels of one 16-byte chunk: four two-element dot products that
// accumulate in float32 (v_dot2c_f32_bf16 / v_dot2c_f32_f16), one instruction per dword where
// taking the halves apart and multiplying them took six.
template <bool BF>
__device__ __forceinline__ float dot8(u32x4 a, u32x4 b) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    float acc = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        // (the dwords are taken out of the vectors as integers first: a bit_cast of a vector
        // element to a 2-vector of 16-bit floats made this compiler read the chunk's first
        // dword four times)
        const uint32_t x = a[j], y = b[j];
        if constexpr (BF)
            acc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, x), __builtin_bit_cast(bf16x2, y), acc, false);
        else
            acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, x), __builtin_bit_cast(f16x2, y), acc, false);
    }
    return acc;
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

// 16 bytes of an output tensor, with a non-temporal store: outputs are written once and
// never read by the kernel that writes them, and stores that do not allocate in L2 leave
// it to the halo rows that neighbouring workgroups share (measured at B4 N4 128x128,
// d=128, k=5: forward 60.9 -> 54.7 us, dQ pass 68.1 -> 61.5, dK/dV pass 96.2 -> 91.4, fused
// backward 147.2 -> 142.7; the same for the read-once query rows was measured slower).
__device__ __forceinline__ void store16(short *p, u32x4 v) {
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}

// Stores one token's D output channels from the accumulators of the second product.
// `acc[t][i]` is channel g*D/4 + t*4 + i of this lane's token (lanes l, l+16, l+32,
// l+48 share a token, g = l/16): D/32 pieces of 16 bytes per lane.  Written as they
// are, a store instruction would put 16-byte pieces D/2 bytes apart (measured at
// D = 128: 3.6 TB/s for a pure write stream of that shape against 5.4 TB/s for 64-byte
// runs).  So at D = 128 the four lanes of a token first exchange pieces with
// v_permlane*_swap (a 4x4 transpose between lane group g and piece number j), and store
// j of the four lanes then covers 64 contiguous bytes.  Every lane of the wave
// must call this; `live` says whether this lane's token exists.  `dlim` is the tensor's
// head dim where it is narrower than the D the kernel is built for (a multiple of 8):
// pieces at or beyond it are not stored.
// LINES (D = 128 only): one more exchange, between the lanes of tokens n and n^1, after which
// every store instruction writes whole 128-byte lines (see below).  It removes the 8-10% of
// extra HBM writes of the 64-byte runs (forward 73.1 -> 68.2 MB, dQ pass 73.5 -> 68.2, dK/dV
// 148.6 -> 134.2, fused backward 222.8 -> 201.4 at B4 N4 128x128) and is used by the kernels
// that run two workgroups per CU, which get 1-9% faster with it (forward 203 -> 194 us at
// 256x256, dQ pass 61.8 -> 56.2, dK/dV 92.6 -> 86.7).  With predicated stores (`live`) the
// kernels with one workgroup per CU get slower (fused backward 118 -> 139 us, dK/dV at k = 7
// 153 -> 165): the branches that the predicates of the exchanged `live` flags put between the
// stores cut the store sequence into blocks that nothing is scheduled across.  Where every
// token exists (ALL: the fused backward, the inner tiles of the dK/dV pass) there are no
// branches and the whole lines cost nothing (fused backward 123.8 -> 122.4 us with them on the
// key side).
// ALL: every lane's token exists (`live` is not looked at), so the stores are not predicated.
template <bool BF, int D, bool LINES = false, bool ALL = false>
__device__ __forceinline__ void store_token(short *token, int g, const f32x4 *acc, float mul,
                                            bool live, int dlim = D) {
    constexpr int NP = D / 32;
    u32x4 p[NP];
#pragma unroll
    for (int j = 0; j < NP; j++) {
        s16x8 w;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            w[i] = cvt16<BF>(acc[2 * j][i] * mul);
            w[4 + i] = cvt16<BF>(acc[2 * j + 1][i] * mul);
        }
        p[j] = __builtin_bit_cast(u32x4, w);
    }
    if constexpr (NP == 4) {
        typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
        // lanes l and l^32 (g bit 1) exchange pieces j and j^2 ...
#pragma unroll
        for (int j0 = 0; j0 < 2; j0++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const u32x2 r = __builtin_amdgcn_permlane32_swap(p[j0][c], p[j0 + 2][c], false, false);
                p[j0][c] = r[0];
                p[j0 + 2][c] = r[1];
            }
        // ... then lanes l and l^16 (g bit 0) pieces j and j^1
#pragma unroll
        for (int j1 = 0; j1 < 2; j1++)
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const u32x2 r =
                    __builtin_amdgcn_permlane16_swap(p[2 * j1][c], p[2 * j1 + 1][c], false, false);
                p[2 * j1][c] = r[0];
                p[2 * j1 + 1][c] = r[1];
            }
        // piece j of this lane is now channels j*D/4 + g*8 .. +8
        if constexpr (LINES) {
            // Stored like that, an instruction would write 64 contiguous bytes per token: half a
            // line, and non-temporal half lines leave L2 before their other half arrives (a pure
            // write stream of 64-byte runs moves 1.42x its bytes at 3.1 TB/s, one of 128-byte runs
            // 1.00x at 5.3 TB/s).  So the lanes of tokens n and n^1 (adjacent lanes) exchange once
            // more: the even lane gives pieces 1 and 3 and takes the odd lane's 0 and 2, and the
            // eight lanes of the pair then write one token's line per instruction.
            const bool odd = threadIdx.x & 1;
            auto xchg = [](unsigned x) __attribute__((always_inline)) {
                return (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true);
            };
            u32x4 s0, s1, s2, s3;
    #pragma unroll
            for (int c = 0; c < 4; c++) {
                const unsigned ra = xchg(odd ? p[0][c] : p[1][c]), rb = xchg(odd ? p[2][c] : p[3][c]);
                s0[c] = odd ? ra : p[0][c];
                s1[c] = odd ? rb : p[2][c];
                s2[c] = odd ? p[1][c] : ra;
                s3[c] = odd ? p[3][c] : rb;
            }
            // (the other token's address as an offset from this one's, so that the stores stay
            // global-memory instructions: an address rebuilt from exchanged integers makes them flat)
            const uintptr_t own = reinterpret_cast<uintptr_t>(token);
            const uintptr_t nbr = (uintptr_t)xchg((unsigned)own) | ((uintptr_t)xchg((unsigned)(own >> 32)) << 32);
            const bool nlive = ALL || xchg(live ? 1u : 0u) != 0;
            short *other = reinterpret_cast<short *>(reinterpret_cast<char *>(token) + (ptrdiff_t)(nbr - own));
            short *tok_a = odd ? other : token, *tok_b = odd ? token : other;
            const bool live_a = ALL || (odd ? nlive : live), live_b = ALL || (odd ? live : nlive);
            const int off = (odd ? 32 : 0) + g * 8;
            if (live_a) {
                if (off < dlim) store16(tok_a + off, s0);
                if (off + 64 < dlim) store16(tok_a + off + 64, s1);
            }
            if (live_b) {
                if (off < dlim) store16(tok_b + off, s2);
                if (off + 64 < dlim) store16(tok_b + off + 64, s3);
            }
        } else if (ALL || live) {
#pragma unroll
            for (int j = 0; j < NP; j++)
                if (j * (D / 4) + g * 8 < dlim) store16(token + j * (D / 4) + g * 8, p[j]);
        }
    } else if constexpr (NP == 2 && LINES) {
        // D = 64: a lane holds 32 contiguous bytes of its token (two pieces), so an instruction
        // writes 16-byte pieces 32 bytes apart.  The lanes of tokens n and n^1 exchange one piece
        // each and the eight lanes of the pair write one token's whole line per instruction.
        const bool odd = threadIdx.x & 1;
        auto xchg = [](unsigned x) __attribute__((always_inline)) {
            return (unsigned)__builtin_amdgcn_mov_dpp((int)x, 0xB1 /* quad_perm [1,0,3,2] */, 0xF, 0xF, true);
        };
        u32x4 s0, s1;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const unsigned r = xchg(odd ? p[0][c] : p[1][c]);
            s0[c] = odd ? r : p[0][c];
            s1[c] = odd ? p[1][c] : r;
        }
        const uintptr_t own = reinterpret_cast<uintptr_t>(token);
        const uintptr_t nbr = (uintptr_t)xchg((unsigned)own) | ((uintptr_t)xchg((unsigned)(own >> 32)) << 32);
        const bool nlive = ALL || xchg(live ? 1u : 0u) != 0;
        short *other = reinterpret_cast<short *>(reinterpret_cast<char *>(token) + (ptrdiff_t)(nbr - own));
        const int off = g * 16 + (odd ? 8 : 0);
        if ((ALL || (odd ? nlive : live)) && off < dlim) store16((odd ? other : token) + off, s0);
        if ((ALL || (odd ? live : nlive)) && off < dlim) store16((odd ? token : other) + off, s1);
    } else {
        // D = 32: the four lanes of a token already cover its 64 bytes.
        if (ALL || live) {
#pragma unroll
            for (int j = 0; j < NP; j++)
                if (g * (D / 4) + j * 8 < dlim) store16(token + g * (D / 4) + j * 8, p[j]);
        }
    }
}

// B operand rows straight from global memory: lane group g takes channels ds*32 + g*8 ..
// of the row at `row` (its channel 0) for ds = 0 .. DS-1.  Chunks at or beyond `dlim`
// (head dims narrower than the kernel's D) are zero and read nothing out of bounds.
template <int DS>
__device__ __forceinline__ void load_row_chunks(s16x8 (&reg)[DS], const short *row, int g, int dlim) {
#pragma unroll
    for (int ds = 0; ds < DS; ds++) {
        const int ch = ds * 32 + g * 8;
        const bool on = ch < dlim;
        const s16x8 v = *reinterpret_cast<const s16x8 *>(row + (on ? ch : 0));
        reg[ds] = on ? v : s16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
}

template <int D, int KS, int NW = 4, int SP = 1>
struct Geo {
    // NW waves own 4x4 pixel blocks, two side by side: a tile of 2*NW x 8 pixels.
    // Four waves (8x8 pixels) everywhere, except that the forward of a configuration
    // whose halo leaves room for only one workgroup per CU can use eight (16x8
    // pixels) where that still fits: two waves per SIMD, and less halo per pixel.
    static constexpr int TH = 2 * NW, TW = 8;     // pixels per workgroup
    // SP waves share each 4x4 block: they split its halo tokens between them and add
    // their partial sums at the end (used where LDS admits one workgroup per CU, so
    // that a SIMD still holds two waves)
    static constexpr int NT = 64 * NW * SP;       // threads per workgroup
    static constexpr int HR = TH + KS - 1;        // halo of the workgroup tile
    static constexpr int HC = TW + KS - 1;
    static constexpr int SW = 4 + KS - 1;         // halo side of one wave's 4x4 block
    // The wave numbers its halo tokens row-major with SWC tokens per row.  SWC is
    // SW, except that a 14-wide halo (k = 11) is numbered 16 per row: 14 * 16 is a
    // multiple of 32 like the padded 14 * 14 would be, so no work is added, and the
    // token -> (row, column) arithmetic becomes shifts (divisions by 14 cost the
    // k = 11 kernels more registers than they have).
    // A 10- or 12-wide halo (k = 7, 9) is numbered in two blocks instead: its first 8
    // columns row-major, 8 per row, then the remaining 2 or 4 columns row-major.  The
    // first block ends on a multiple of 16 tokens, so for every 16-token tile the
    // (row, column) of a token is shifts and masks of its number (tok_rc): divisions by
    // 10 or 12 cost those kernels up to 80 registers of hoisted quotients.
    static constexpr int SWC = SW == 14 ? 16 : SW;
    static constexpr int W1 = (SW == 10 || SW == 12) ? 8 : 0;
    static constexpr int NK = SW * SWC;           // token numbers per wave (some unused)
    // (row, column) in the wave's halo of token tile * 16 + x, x in [0, 16); false: no
    // such token.  `tile` is a compile-time constant wherever this is called.
    static __device__ __forceinline__ bool tok_rc(int tile, int x, int &r, int &c) {
        if constexpr (W1 != 0) {
            constexpr int A_TILES = SW * W1 / 16, W2 = SW - W1;
            if (tile < A_TILES) {
                const int tk = tile * 16 + x;
                r = tk >> 3;
                c = tk & 7;
                return true;
            }
            const int tb = (tile - A_TILES) * 16 + x;
            r = tb / W2;
            c = W1 + tb % W2;
            return r < SW;
        } else {
            const int tk = tile * 16 + x;
            r = tk / SWC;
            c = tk % SWC;
            return tk < NK && c < SW;
        }
    }
    // token tile * 16 + x lies in the k x k window that starts at (dr, dc) of the halo
    template <int K>
    static __device__ __forceinline__ bool tok_in(int tile, int x, int dr, int dc) {
        int r, c;
        const bool ok = tok_rc(tile, x, r, c);
        return ok && (unsigned)(r - dr) < (unsigned)K && (unsigned)(c - dc) < (unsigned)K;
    }
    static constexpr int NKP = (NK + 31) / 32 * 32;
    static constexpr int MT = NKP / 16;           // 16-token MFMA row tiles
    static constexpr int KSTEPS = NKP / 32;       // reduction steps of the second product
    // LDS layout.  A row holds the D channels of one pixel.  Two layouts are written
    // down; SWZ picks one at compile time and every address goes through the helpers
    // below, which fold to plain constants for the padded layout.
    //  * padded (SWZ = false): rows D + 8 elements apart.  The rows of an MFMA operand
    //    tile (one row per lane, the same 16-byte chunk of each) then start 4 banks
    //    apart; a 16-byte operand read costs 12 LDS cycles against 8.3 for a conflict-free
    //    one (measured on the token pattern of kernel_size 5).
    //  * swizzled (SWZ = true): rows D elements apart, chunk c of row r kept at chunk
    //    position c ^ key(r), where key(r) runs through all CPR values over the rows that
    //    share one 256-byte line of the 64 banks and the lines after it.  Operand reads
    //    are then conflict-free and LDS holds 6-20% more pixels, but every read address
    //    needs an XOR with a per-lane value instead of a constant offset: at head_dim 128,
    //    kernel_size 5 the forward, dQ and dK/dV kernels execute 27% more vector
    //    instructions with it, LDS conflict cycles fall from 44-52% to 34-39% of the LDS
    //    cycles, and the kernels get 3-5% SLOWER (they wait on memory and instruction
    //    latency, not on LDS bandwidth, which is about a third used).  So it is off.
    static constexpr bool SWZ = false;
    static constexpr int PITCH = SWZ ? D : D + 8;  // LDS row pitch in elements
    static constexpr int ROWS = HR * HC + 1;      // + one all-zero row for padding tokens
    static constexpr int ZROW = HR * HC;
    static constexpr int CPR = D / 8;             // 16-byte chunks per row
    static constexpr int RPL = 16 / CPR;          // rows per 256-byte line (1, 2 or 4)
    static constexpr int LB = D == 128 ? 2 : D == 64 ? 1 : 0;  // log2(D / 32)
    static __device__ __forceinline__ int key(int row) { return SWZ ? (row / RPL) & (CPR - 1) : 0; }
    // element offset of chunk c of a row
    static __device__ __forceinline__ int chunk_at(int row, int c) {
        return row * PITCH + ((c ^ key(row)) << 3);
    }
    // A operand of the first products: lane group g reads chunk g + 4 * ds of its row for
    // ds = 0 .. DS-1.  a_row gives the address for ds = 0 up to the XOR with the high part
    // of the key, a_at the address for a given (compile-time) ds.
    struct ARow { const short *p; int kh; };
    static __device__ __forceinline__ ARow a_row(const short *lds, int row, int g) {
        const int k = key(row);
        return ARow{lds + row * PITCH + ((g ^ (k & 3)) << 3), k >> 2};
    }
    static __device__ __forceinline__ const short *a_at(const ARow &r, int ds) {
        return r.p + ((ds ^ r.kh) << 5);
    }
    // A operand of the second products (transposing reads): lane n reads 4 elements at
    // element (n & 3) * D/4 + mt * 4 of its row for mt = 0 .. DT-1, i.e. chunk
    // ((n & 3) << LB) | (mt >> 1), half (mt & 1).
    struct TRow { const short *p; int kl; };
    static __device__ __forceinline__ TRow t_row(const short *lds, int row, int n) {
        const int k = key(row);
        return TRow{lds + row * PITCH + ((((n & 3) ^ (k >> LB)) << LB) << 3), k & ((1 << LB) - 1)};
    }
    static __device__ __forceinline__ const short *t_at(const TRow &r, int mt) {
        return r.p + ((((mt >> 1) ^ r.kl) << 3) | ((mt & 1) << 2));
    }
    static constexpr int DS = D / 32;             // reduction steps over channels
    static constexpr int DT = D / 16;             // 16-channel MFMA row tiles of the output
    static constexpr int NCH = HR * HC * CPR;     // 16-byte chunks per staged halo
    static constexpr int NL = (NCH + NT - 1) / NT;  // chunks per thread
    static constexpr int NST = (ROWS + NT - 1) / NT;  // per-query statistics per thread
    static constexpr size_t LDS_BYTES =
        (size_t)2 * ROWS * PITCH * sizeof(short) + ROWS * 2 * sizeof(float);
    // waves per SIMD to budget registers for: one per workgroup that LDS admits
    // on a CU (a workgroup puts one wave on each of the four SIMDs), at most 2
    static constexpr int WAVES = NW == 4 && SP == 1 ? (2 * LDS_BYTES <= 160 * 1024 ? 2 : 1) : 2;
    // staged LDS row of wave token tile * 16 + x whose halo starts at (orow, ocol) of the
    // staged block; numbers that are no token read the all-zero row
    static __device__ __forceinline__ int token_row(int tile, int x, int orow, int ocol) {
        int r, c;
        return tok_rc(tile, x, r, c) ? (orow + r) * HC + ocol + c : (int)ZROW;
    }
    // the same when the rows of the staged block are kept in LDS cyclically: image
    // row y of the block sits in row slot y % HR, and rot = (first image row of the
    // block) % HR
    static __device__ __forceinline__ int token_row_rot(int tile, int x, int orow, int ocol, int rot) {
        int r, c;
        const bool ok = tok_rc(tile, x, r, c);
        int y = orow + r + rot;
        y = y >= HR ? y - HR : y;
        return ok ? y * HC + ocol + c : (int)ZROW;
    }
};

// Persistent, XCD-aware tile schedule.  Hardware deals consecutive workgroup ids
// round-robin to the 8 XCDs, each with its own L2: every XCD gets one contiguous
// run of tiles, and the workgroups resident on it sweep that run side by side, so
// the halos shared by neighbouring tiles meet in the same L2.
struct Sched {
    int t, t_end, step;
    int seg_end, skip, hop;  // see make_runs; a strided walk has one endless segment
};
__device__ __forceinline__ Sched make_sched(int ntiles, int block, int nblocks) {
    const int xcd = block & 7, slot = block >> 3, slots = nblocks >> 3;
    const int per = (ntiles + 7) >> 3;
    Sched sc;
    sc.t = xcd * per + slot;
    sc.t_end = min(ntiles, (xcd + 1) * per);
    sc.step = slots;
    sc.seg_end = 0x7fffffff; sc.skip = 0; sc.hop = 0;
    return sc;
}

// The same split over the XCDs, but a workgroup takes contiguous segments of its
// XCD's tiles.  With tiles numbered down the columns of an image (tile_of_cm) a
// workgroup then walks down a column, and consecutive tiles share k-1 of their
// halo's rows, which stay in LDS.  `per` tiles go to each XCD, in segments of `seg`
// tiles; the workgroups of an XCD take segment after segment in turn, so that at
// any time they are at work on neighbouring columns (or neighbouring parts of one)
// and the halo columns those share meet in the XCD's L2.  Host side: plan_runs.
struct Runs {
    int per, seg;
};
__device__ __forceinline__ Sched make_runs(int ntiles, int block, int nblocks, Runs rp) {
    const int xcd = block & 7, slot = block >> 3, slots = nblocks >> 3;
    const int lo = xcd * rp.per;
    Sched sc;
    sc.t = lo + slot * rp.seg;
    sc.t_end = min(ntiles, lo + rp.per);
    sc.step = 1;
    sc.seg_end = sc.t + rp.seg;
    sc.hop = slots * rp.seg;
    sc.skip = sc.hop - rp.seg;
    return sc;
}
// the tile after sc.t (at or beyond sc.t_end: none), and the step to it
__device__ __forceinline__ int sched_peek(const Sched &sc) {
    const int tn = sc.t + sc.step;
    return tn >= sc.seg_end ? tn + sc.skip : tn;
}
__device__ __forceinline__ void sched_advance(Sched &sc, int tn) {
    if (tn >= sc.seg_end) sc.seg_end += sc.hop;
    sc.t = tn;
}

struct Tile {
    int bb, nn, r0, c0;
};
__device__ __forceinline__ Tile tile_of_cm(int t, int tiles_r, int tiles_c, int N) {
    Tile tl;
    tl.r0 = (t % tiles_r) * 8; t /= tiles_r;
    tl.c0 = (t % tiles_c) * 8; t /= tiles_c;
    tl.bb = t / N; tl.nn = t % N;
    return tl;
}
__device__ __forceinline__ Tile tile_of(int t, int tiles_r, int tiles_c, int N, int th = 8) {
    Tile tl;
    tl.c0 = (t % tiles_c) * 8; t /= tiles_c;
    tl.r0 = (t % tiles_r) * th; t /= tiles_r;
    tl.bb = t / N; tl.nn = t % N;
    return tl;
}

// Staging plan of one thread: which 16-byte chunks of a halo it moves.  Chunk i of
// thread t is chunk number t + 256*i of the halo in (row, column, channel-chunk)
// order.  The plan is the same for every tile, so it is computed once.
template <int D, int KS, int NW = 4, int SP = 1>
struct HaloPlan {
    int rc[Geo<D, KS, NW, SP>::NL];  // halo row << 8 | halo column of chunk i
    int ch8;                 // first channel of the thread's chunks
    int lds0;                // LDS element offset of chunk 0
    bool on;                 // false: the tensor has no such channels (head dim below D); the
                             // thread moves nothing and its LDS columns stay zero (zero_row)
};
template <int D, int KS, int NW = 4, int SP = 1>
__device__ __forceinline__ HaloPlan<D, KS, NW, SP> make_plan(int dlim = D) {
    using G = Geo<D, KS, NW, SP>;
    static_assert(G::NT % G::CPR == 0, "a thread keeps one channel chunk");
    HaloPlan<D, KS, NW, SP> pl;
    pl.ch8 = (threadIdx.x % G::CPR) * 8;
    pl.on = pl.ch8 < dlim;
    // the rows of one thread's chunks are NT / CPR apart, a multiple of 16 * RPL, so they
    // share one key and the chunk position is the same for all of them
    static_assert((G::NT / G::CPR) % (16 * G::RPL) == 0, "one chunk position per thread");
    pl.lds0 = G::chunk_at(threadIdx.x / G::CPR, threadIdx.x % G::CPR);
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        int row = threadIdx.x / G::CPR + i * (G::NT / G::CPR);
        row = row < G::HR * G::HC ? row : G::HR * G::HC - 1;  // tail: harmless duplicate
        pl.rc[i] = ((row / G::HC) << 8) | (row % G::HC);
    }
    return pl;
}
template <int D, int KS, int NW = 4, int SP = 1>
struct HaloRegs {
    u32x4 v[Geo<D, KS, NW, SP>::NL];
};
// Global -> registers: this thread's share of the halo with origin (hr0, hc0) of
// one image.  Halo positions at or beyond (rlim, clim) are not needed by any
// unmasked product; they are clamped to the last valid row / column so the loads
// stay in bounds and branch-free (the values only ever meet zero probabilities).
// Addresses are a uniform base plus a 32-bit per-lane byte offset formed with
// 24-bit multiplies: strides are below 2^22 elements (checked on the host).
// (I0, I1: only this thread's chunks I0 .. I1-1, for a kernel that loads the last chunks of a
// halo behind its arithmetic because it has no registers for them beside it)
template <int D, int KS, int NW = 4, int SP = 1, int I0 = 0, int I1 = Geo<D, KS, NW, SP>::NL>
__device__ __forceinline__ void halo_fetch(HaloRegs<D, KS, NW, SP> &reg, const HaloPlan<D, KS, NW, SP> &pl,
                                  const short *img, int64_t sh, int64_t sw, int hr0, int hc0,
                                  int rlim, int clim) {
    using G = Geo<D, KS, NW, SP>;
    const char *base = reinterpret_cast<const char *>(img + hr0 * sh + hc0 * sw);
    const unsigned sh2 = (unsigned)sh * 2u, sw2 = (unsigned)sw * 2u;
    const int rmax = rlim - 1 - hr0, cmax = clim - 1 - hc0;
    if (!pl.on) return;
#pragma unroll
    for (int i = I0; i < I1; i++) {
        const unsigned r = (unsigned)min(pl.rc[i] >> 8, rmax);
        const unsigned c = (unsigned)min(pl.rc[i] & 255, cmax);
        const unsigned off = __umul24(r, sh2) + __umul24(c, sw2) + (unsigned)pl.ch8 * 2u;
        reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off);
    }
}
// Registers -> LDS, one row of D channels per pixel, chunks permuted (Geo::key).
template <int D, int KS, int NW = 4, int SP = 1>
__device__ __forceinline__ void halo_commit(short *lds, const HaloPlan<D, KS, NW, SP> &pl,
                                   const HaloRegs<D, KS, NW, SP> &reg) {
    using G = Geo<D, KS, NW, SP>;
    if (!pl.on) return;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        const int row = threadIdx.x / G::CPR + i * (G::NT / G::CPR);
        if (row < G::HR * G::HC)
            *reinterpret_cast<u32x4 *>(lds + pl.lds0 + i * (G::NT / G::CPR) * G::PITCH) = reg.v[i];
    }
}
// Row-range variants for halos whose rows are kept in LDS cyclically (image row y
// in row slot y % HR): move only the `nrows` image rows from y0 on, all HC columns
// from hc0 on.  A tile that follows its upper neighbour thus loads only the rows
// the neighbour's halo did not hold.
template <int D, int KS, int NW = 4, int SP = 1>
__device__ __forceinline__ void halo_fetch_rows(HaloRegs<D, KS, NW, SP> &reg, const HaloPlan<D, KS, NW, SP> &pl,
                                                const short *img, int64_t sh, int64_t sw, int y0,
                                                int hc0, int nrows, int rlim, int clim) {
    using G = Geo<D, KS, NW, SP>;
    const int yb = min(y0, rlim - 1);
    const char *base = reinterpret_cast<const char *>(img + yb * sh + hc0 * sw);
    const unsigned sh2 = (unsigned)sh * 2u, sw2 = (unsigned)sw * 2u;
    const int rmax = rlim - 1 - yb, cmax = clim - 1 - hc0;
    if (!pl.on) return;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        const int r = pl.rc[i] >> 8;
        if (r < nrows) {
            const unsigned rr = (unsigned)min(r, rmax);
            const unsigned c = (unsigned)min(pl.rc[i] & 255, cmax);
            const unsigned off = __umul24(rr, sh2) + __umul24(c, sw2) + (unsigned)pl.ch8 * 2u;
            reg.v[i] = *reinterpret_cast<const u32x4 *>(base + off);
        }
    }
}
template <int D, int KS, int NW = 4, int SP = 1>
__device__ __forceinline__ void halo_commit_rows(short *lds, const HaloPlan<D, KS, NW, SP> &pl,
                                                 const HaloRegs<D, KS, NW, SP> &reg, int y0, int nrows) {
    using G = Geo<D, KS, NW, SP>;
    const int rot = y0 % G::HR;
    if (!pl.on) return;
#pragma unroll
    for (int i = 0; i < G::NL; i++) {
        const int pix = threadIdx.x / G::CPR + i * (G::NT / G::CPR);
        const int r = pl.rc[i] >> 8;
        if (pix < G::HR * G::HC && r < nrows) {
            int slot = rot + r;
            slot = slot >= G::HR ? slot - G::HR : slot;
            *reinterpret_cast<u32x4 *>(lds + G::chunk_at(slot * G::HC + (pl.rc[i] & 255),
                                                          threadIdx.x % G::CPR)) = reg.v[i];
        }
    }
}
// The spare row stays zero for the whole kernel: padding tokens and tokens
// outside a wave's halo read it, so they add exact zeros to the second product.
// With a head dim below D (`dlim`), the channels from it on are zeroed in EVERY row, once:
// no commit writes them (HaloPlan::on), so they stay zero as long as nothing else is laid
// over the rows.
template <int D, int KS, int NW = 4, int SP = 1>
__device__ __forceinline__ void zero_row(short *lds, int dlim = D) {
    using G = Geo<D, KS, NW, SP>;
    if (threadIdx.x < G::CPR)
        *reinterpret_cast<uint4 *>(lds + G::ZROW * G::PITCH + threadIdx.x * 8) =  // all zero: any order
            make_uint4(0, 0, 0, 0);
    if (dlim < D) {
        static_assert(!G::SWZ, "the padding columns are the last chunks of a row");
        const int c0 = dlim >> 3, npad = G::CPR - c0;
        for (int idx = threadIdx.x; idx < G::ZROW * npad; idx += G::NT)
            *reinterpret_cast<uint4 *>(lds + (idx / npad) * G::PITCH + (c0 + idx % npad) * 8) =
                make_uint4(0, 0, 0, 0);
    }
}

// What one lane needs to know about its query (forward, dQ) inside a tile.
struct LaneQ {
    bool wave_on, live;
    int qr, qc;      // query pixel, clamped into the image
    int orow, ocol;  // origin of the wave's halo inside the staged halo
    int dr, dc;      // window start of this query relative to the wave's halo
    int hr0, hc0;    // origin of the staged halo in the image
    int64_t tok;     // flat token index of the query
};
template <int KS>
__device__ __forceinline__ LaneQ lane_query(const Tile &tl, const Shape &s, int wave, int n) {
    LaneQ q;
    const int wr0 = tl.r0 + (wave >> 1) * 4, wc0 = tl.c0 + (wave & 1) * 4;
    q.wave_on = wr0 < s.H && wc0 < s.W;
    q.live = (wr0 + (n >> 2) < s.H) && (wc0 + (n & 3) < s.W);
    q.qr = min(wr0 + (n >> 2), s.H - 1);
    q.qc = min(wc0 + (n & 3), s.W - 1);
    q.hr0 = win_start(tl.r0, s.H, KS);
    q.hc0 = win_start(tl.c0, s.W, KS);
    const int sr0 = win_start(min(wr0, s.H - 1), s.H, KS);
    const int sc0 = win_start(min(wc0, s.W - 1), s.W, KS);
    q.orow = sr0 - q.hr0;
    q.ocol = sc0 - q.hc0;
    q.dr = win_start(q.qr, s.H, KS) - sr0;
    q.dc = win_start(q.qc, s.W, KS) - sc0;
    q.tok = (((int64_t)tl.bb * s.N + tl.nn) * s.H + q.qr) * s.W + q.qc;
    return q;
}

template <typename T>
__device__ __forceinline__ const short *image(const View &v, const Tile &tl) {
    return static_cast<const short *>(v.ptr) + tl.bb * v.sb + tl.nn * v.sn;
}

__device__ __forceinline__ Tile inner_tile(int t, const TileSet &ts, int N) {
    Tile tl;
    tl.c0 = (ts.ic0 + t % ts.ni_c) * 8; t /= ts.ni_c;
    tl.r0 = (ts.ir0 + t % ts.ni_r) * 8; t /= ts.ni_r;
    tl.bb = t / N; tl.nn = t % N;
    return tl;
}
// inner tiles numbered down the columns of the inner rectangle
__device__ __forceinline__ Tile inner_tile_cm(int t, const TileSet &ts, int N) {
    Tile tl;
    tl.r0 = (ts.ir0 + t % ts.ni_r) * 8; t /= ts.ni_r;
    tl.c0 = (ts.ic0 + t % ts.ni_c) * 8; t /= ts.ni_c;
    tl.bb = t / N; tl.nn = t % N;
    return tl;
}
__device__ __forceinline__ Tile frame_tile(int t, const TileSet &ts, int N) {
    const int per_img = ts.tiles_r * ts.tiles_c - ts.ni_r * ts.ni_c;
    const int slab = t / per_img;
    int e = t % per_img;
    const int top = ts.ir0 * ts.tiles_c, side = ts.tiles_c - ts.ni_c;
    int tr, tc;
    if (e < top) {
        tr = e / ts.tiles_c; tc = e % ts.tiles_c;
    } else if (e < top + ts.ni_r * side) {
        e -= top;
        tr = ts.ir0 + e / side;
        tc = e % side;
        tc = tc < ts.ic0 ? tc : tc + ts.ni_c;
    } else {
        e -= top + ts.ni_r * side;
        tr = ts.ir0 + ts.ni_r + e / ts.tiles_c; tc = e % ts.tiles_c;
    }
    Tile tl;
    tl.r0 = tr * 8; tl.c0 = tc * 8;
    tl.bb = slab / N; tl.nn = slab % N;
    return tl;
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
           v.sh % 8 == 0 && v.sw % 8 == 0 && v.sh < (1 << 22) && v.sw < (1 << 22);
}

// Persistent grid: as many workgroups as stay resident at once (8 XCDs x 32 CUs x
// workgroups per CU), never more than there are tiles.  The occupancy of a kernel
// is queried once; the kernel is a template argument so that every instantiation
// has its own cached value (kernels of one signature share a function type).
template <auto KERNEL>
int persistent_grid(int64_t ntiles, int threads = 256) {
    static const int per_cu = [threads]() {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, KERNEL, threads, 0) != hipSuccess || n < 1)
            n = 1;
        return n;
    }();
    const int64_t per_xcd = (ntiles + 7) / 8;
    const int64_t slots = per_xcd < 32 * (int64_t)per_cu ? per_xcd : 32 * (int64_t)per_cu;
    return (int)(8 * slots);
}

// Segments for make_runs.  While a workgroup's share is at most one column (`colh`
// tiles) it is one segment.  Several columns in a row would put the workgroups of
// an XCD on columns that are never neighbours at the same time; then the segments
// are whole columns, or equal parts of a column, dealt out in turn, chosen for the
// shortest walk of the busiest workgroup (a segment start costs about half a tile:
// the whole halo is staged, not 8 rows of it).  `walk`, if given, receives that walk in
// half tiles.
inline Runs plan_runs(int64_t ntiles, int grid, int colh, double *walk = nullptr) {
    const int64_t slots = grid / 8, per = (ntiles + 7) / 8;
    const int64_t run = (per + slots - 1) / slots;
    Runs rp{(int)per, (int)run};
    double best = 2.0 * run + 1.0;
    if (walk) *walk = best;
    if (run <= colh) return rp;
    best *= 1.3;  // measured: without the shared L2 lines, 1.3x the time
    for (int m = 1; m <= 8; m++) {
        if (colh % m) continue;
        const int64_t seg = colh / m;
        const int64_t per_a = (per + seg - 1) / seg * seg;
        const int64_t rounds = (per_a + slots * seg - 1) / (slots * seg);
        const double cost = rounds * (2.0 * seg + 1.0);
        if (cost < best) {
            best = cost;
            rp.per = (int)per_a;
            rp.seg = (int)seg;
        }
    }
    if (walk) *walk = best;
    return rp;
}

}  // namespace
}  // namespace enatten
