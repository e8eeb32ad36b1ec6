// Shared declarations of the neighborhood-attention kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "enatten.h"

namespace enatten {

// A [B, heads, H, W, D] tensor with unit stride on D; strides in elements.
struct View {
    const void *ptr;
    int64_t sb, sn, sh, sw;
};

struct Shape {
    int B, N, H, W, D;
    int kh, kw;  // window extent on rows / columns (kh == kw for the reference's operator)
    float scale;
    int ch, cw;  // causal rows / columns: a query only sees keys at or before it on that axis
};

struct FwdArgs {
    View q, k, v;
    View o;      // written; same kind of strided view as q, k, v
    float *lse;  // contiguous [B, N, H, W] or nullptr
    Shape s;
    const void *rpb = nullptr;  // relative position bias [N, 2*kh-1, 2*kw-1] in the tensors' type
};

struct BwdArgs {
    View q, k, v;
    View o, d_o;  // forward output and upstream gradient, strided views like q, k, v
    const float *lse;
    void *dq, *dk, *dv;
    // element strides of dq, dk and dv alike on (batch, head, row, column), unit stride on the
    // channels: contiguous tensors unless the caller writes the gradients into strided views
    // (the sub-grids of a dilated call); set_grad_layout fills them
    int64_t gsb, gsn, gsh, gsw;
    __host__ __device__ int64_t grad_at(int b, int n, int y, int x) const {
        return b * gsb + n * gsn + y * gsh + x * gsw;
    }
    bool grads_contiguous() const {
        return gsw == s.D && gsh == (int64_t)s.W * s.D && gsn == (int64_t)s.H * s.W * s.D &&
               gsb == (int64_t)s.N * s.H * s.W * s.D;
    }
    float *delta;        // scratch [B, N, H, W]: sum_j P_j dP_j per query
    float *zinv;         // scratch [B, N, H, W]: 1 / sum_j exp(S_j - lse) (vector-ALU kernels)
    Shape s;
    const void *rpb = nullptr;  // relative position bias [N, 2*kh-1, 2*kw-1] in the tensors' type
    float *d_rpb = nullptr;     // its gradient, float32, fully overwritten (general kernels)
    float *ds_pairs = nullptr;  // scratch [B, N, H, W, kh*kw]: dS of every (query, window position),
                                // from which d_rpb is summed in a fixed order
};

// NATTEN window start on an axis of length L: centred, shifted to stay inside
// (e_natten/pytorch.py:7-11, e_natten/triton.py:7-12).
__host__ __device__ inline int win_start(int i, int L, int k) {
    int s = i - (k >> 1);
    s = s < 0 ? 0 : s;
    return s > L - k ? L - k : s;
}
// Queries whose window contains key i form [inv_lo, inv_hi)
// (e_natten/pytorch.py:13-23).
__host__ __device__ inline int inv_lo(int i, int k) { return i < k ? 0 : i - (k >> 1); }
__host__ __device__ inline int inv_hi(int i, int L, int k) {
    return i >= L - k ? L : i + (k >> 1) + 1;
}

// The same rules with the causal variant of an axis (NATTEN's causal neighbourhood: the
// last k positions up to and including the query's own, fewer at the start of the axis;
// the reference has no causal mode).  A query at i sees keys [axis_start, axis_start +
// axis_count); a key at j is seen by the queries [axis_inv_lo, axis_inv_hi).
__host__ __device__ inline int axis_start(int i, int L, int k, int causal) {
    return causal ? (i - k + 1 < 0 ? 0 : i - k + 1) : win_start(i, L, k);
}
__host__ __device__ inline int axis_count(int i, int L, int k, int causal) {
    return causal ? i - axis_start(i, L, k, 1) + 1 : k;
}
__host__ __device__ inline int axis_inv_lo(int j, int k, int causal) {
    return causal ? j : inv_lo(j, k);
}
__host__ __device__ inline int axis_inv_hi(int j, int L, int k, int causal) {
    return causal ? (j + k < L ? j + k : L) : inv_hi(j, L, k);
}

// The 8x8 tiles of an image split into an inner rectangle, where no key or query
// is within reach of the border, and the frame around it.
struct TileSet {
    int tiles_r, tiles_c;  // 8x8 tiles per image
    int ir0, ni_r;         // first inner tile row, number of inner tile rows
    int ic0, ni_c;         // first inner tile column, number of inner tile columns
};

void set_error(const char *fmt, ...);

// Brackets one kernel launch with HIP events while the timing aid is enabled
// (enatten_prof.cpp); does nothing, and touches no shared state, while it is off.
struct ProfScope {
    int slot;
    hipStream_t st;
    hipEvent_t e0, e1, e2;
    unsigned generation;
    bool armed;
    ProfScope(int kernel_slot, const char *kernel_name, hipStream_t stream);
    ~ProfScope();
    ProfScope(const ProfScope &) = delete;
    ProfScope &operator=(const ProfScope &) = delete;
};

// general fp32-FMA kernels: any D <= 1024, any odd window, f32 / bf16 / f16
int launch_fwd_simt(const FwdArgs &a, int dtype, hipStream_t st);
int launch_bwd_simt(const BwdArgs &a, int dtype, hipStream_t st);

// float64 tensors (plain double arithmetic; windows as the general kernels, no bias).  The
// backward keeps two doubles per query in a.delta (16-byte aligned).
int launch_fwd_f64(const FwdArgs &a, hipStream_t st);
int launch_bwd_f64(const BwdArgs &a, hipStream_t st);

// float32 matrix-core kernels (float64 logits): D in {32, 64, 128}, kernel_size 3 / 5 / 7.
// Their backward keeps 2 * ks * ks float32 per query in the workspace (a.delta).
bool mfma_f32_supported(int D, int ks, int dtype);
size_t mfma_f32_workspace_floats(int ks);
int launch_fwd_mfma_f32(const FwdArgs &a, hipStream_t st);
int launch_bwd_mfma_f32(const BwdArgs &a, hipStream_t st);

// matrix-core kernels: bf16 / f16, D in {32, 64, 128}, square odd window
bool mfma_supported(int D, int ks, int dtype);
int launch_fwd_mfma(const FwdArgs &a, int dtype, hipStream_t st);
// `path`: 0 chooses between the two-pass and the fused backward, ENATTEN_PATH_MFMA_FUSED /
// ENATTEN_PATH_MFMA_SPLIT force one of them (ENATTEN_PATH_MFMA_SPLIT_QUEUE: the two passes,
// the dK/dV pass dealing its frame tiles from a counter)
inline bool split_forced(int path) {
    return path == ENATTEN_PATH_MFMA_SPLIT || path == ENATTEN_PATH_MFMA_SPLIT_QUEUE;
}
int launch_bwd_mfma(const BwdArgs &a, int dtype, int path, hipStream_t st);
// the same kernels built for head dims that are multiples of 8 below the next of 32, 64, 128
int launch_fwd_mfma_narrow(const FwdArgs &a, int dtype, hipStream_t st);
int launch_bwd_mfma_narrow(const BwdArgs &a, int dtype, int path, hipStream_t st);
// matrix-core kernels of the 1D operator (a.s: H = 1, W = T, kh = 1, kw = kernel_size):
// bf16 / f16, D in {32, 64, 128}, odd kernel_size 3 .. 49
bool mfma1d_supported(int D, int ks, int dtype);
int launch_fwd1d_mfma(const FwdArgs &a, int dtype, hipStream_t st);
int launch_bwd1d_mfma(const BwdArgs &a, int dtype, int path, hipStream_t st);
int launch_fwd1d_mfma_narrow(const FwdArgs &a, int dtype, hipStream_t st);
int launch_bwd1d_mfma_narrow(const BwdArgs &a, int dtype, int path, hipStream_t st);
// fused backward (dQ, dK, dV of every tile from one staging), where built
bool fused_bwd_supported(const BwdArgs &a);
int launch_bwd_fused(const BwdArgs &a, bool bf16, const TileSet &ts, int64_t ntiles,
                     hipStream_t st);

// one-pass backward of the configurations whose block of all four inputs fits LDS twice
// per CU (head_dim 32 with kernel_size <= 7, head_dim 64 with kernel_size 3)
bool onepass_bwd_supported(const BwdArgs &a);
int launch_bwd_onepass(const BwdArgs &a, bool bf16, const TileSet &ts, int64_t ntiles,
                       hipStream_t st);

}  // namespace enatten
