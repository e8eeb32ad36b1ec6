/*
 * enatten.h - C ABI of the MI355X (gfx950) neighborhood-attention library.
 *
 * One shared library, libenatten.so, exports exactly the functions declared
 * here.  Every function takes raw device pointers, sizes and a HIP stream; none
 * allocates, frees, synchronises or throws.  A non-zero return value is an error
 * code and enatten_last_error() describes it (per calling thread).
 *
 * Tensor layout: [B, heads, H, W, D] as in the reference
 * (e_natten/triton.py:489-518).  The last axis has stride 1.  q, k, v, the forward
 * output o and the upstream gradient d_o may be strided views, as in the reference,
 * which passes the strides of each of them to its kernels
 * (e_natten/triton.py:509-512, :539-545): their element strides for the (batch,
 * head, row, column) axes are passed as int64_t[4]; NULL means contiguous.  The
 * gradients dq, dk, dv, the log-sum-exp and the workspace are contiguous.  The logits
 * are q.k * scale; the reference applies no scale (e_natten/triton.py:280), so
 * drop-in callers pass 1.0f.
 */
#ifndef ENATTEN_H
#define ENATTEN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ENATTEN_ABI_VERSION 5

/* element types of q, k, v, o and the gradients.  ENATTEN_F64 runs in plain double
 * arithmetic on kernels of its own (for numerical gradient checks, as the reference's
 * gradcheck.py:6-15 does; not tuned); lse stays float32. */
enum { ENATTEN_F32 = 0, ENATTEN_BF16 = 1, ENATTEN_F16 = 2, ENATTEN_F64 = 3 };

/* return codes */
enum {
    ENATTEN_OK = 0,
    ENATTEN_EINVAL = 1,       /* bad shape, kernel size, stride, pointer or dtype */
    ENATTEN_EUNSUPPORTED = 2, /* valid request outside what the kernels cover */
    ENATTEN_ELAUNCH = 3       /* the HIP runtime refused the launch */
};

/* which kernel family a call is routed to (enatten2d_kernel_path) */
enum { ENATTEN_PATH_NONE = 0, ENATTEN_PATH_SIMT = 1, ENATTEN_PATH_MFMA = 2,
       ENATTEN_PATH_MFMA_FUSED = 3, ENATTEN_PATH_MFMA_SPLIT = 4 /* enatten_set_path only */,
       ENATTEN_PATH_MFMA_SPLIT_QUEUE = 5 /* enatten_set_path only */ };

int enatten_abi_version(void);

/* Message for the last non-zero return code on this thread ("" if none). */
const char *enatten_last_error(void);

/*
 * Kernel family that would serve (D, kernel_size, dtype): ENATTEN_PATH_MFMA for
 * the matrix-core kernels, ENATTEN_PATH_SIMT for the general fp32-FMA kernels,
 * ENATTEN_PATH_NONE if the call would be rejected.
 */
int enatten2d_kernel_path(int D, int kernel_size, int dtype);

/*
 * Steer dispatch: 0 = automatic (default), ENATTEN_PATH_SIMT = never use the
 * matrix-core kernels.  The matrix-core backward has two forms: two passes (dQ, then
 * dK/dV) and one fused kernel that stages q, k, v, dO once (built for head_dim 128,
 * kernel_size 5, image sides that are multiples of 8; the 1D operator has one for
 * kernel_size <= 17, and for head_dim <= 64 beyond).  Automatic dispatch and
 * ENATTEN_PATH_MFMA_FUSED take the fused form wherever it is built (it was measured
 * faster at every size), ENATTEN_PATH_MFMA_SPLIT never.  ENATTEN_PATH_MFMA_SPLIT_QUEUE is
 * ENATTEN_PATH_MFMA_SPLIT with the dK/dV pass dealing its border tiles from a counter as
 * workgroups become free wherever it has any (automatic dispatch does that where its cost
 * model says it pays).
 * Process-wide; meant for tests and tuning.  Returns the previous setting.
 */
int enatten_set_path(int path);

/*
 * Forward of 2D neighborhood attention.
 * Replaces the launch of _attn_fwd_2d in Natten2d.forward
 * (e_natten/triton.py:507-513; per-query math triton.py:242-302, CPU statement
 * e_natten/pytorch.py:178-202).
 *
 *   o   [B, heads, H, W, D]  dtype, every element overwritten; o_strides lets the
 *                            caller have it written straight into, say, a
 *                            [B, H, W, heads, D] buffer
 *   lse [B, heads, H, W]     float32 natural-log sum-exp of each query's scaled
 *                            logits, contiguous; may be NULL if no backward
 *                            will follow
 * kernel_size is odd, 1 <= kernel_size <= min(H, W).
 */
int enatten2d_fwd(const void *q, const void *k, const void *v, void *o, float *lse,
                  int B, int heads, int H, int W, int D, int kernel_size, int dtype,
                  const int64_t *q_strides, const int64_t *k_strides,
                  const int64_t *v_strides, const int64_t *o_strides, float scale,
                  void *stream);

/*
 * Bytes of device scratch enatten2d_bwd needs for a call of this shape: two float32
 * per query, or 2 * kernel_size^2 per query where the float32 matrix-core kernels
 * serve the call (they hand the probabilities and their gradients from the dQ pass to
 * the dK/dV pass through it), or two doubles per query for float64 tensors (16-byte
 * aligned).
 */
size_t enatten2d_bwd_workspace_bytes(int B, int heads, int H, int W, int D, int kernel_size,
                                     int dtype);

/*
 * Backward of 2D neighborhood attention.
 * Replaces the launch of _attn_bwd_2d in Natten2d.backward
 * (e_natten/triton.py:537-546; per-query math triton.py:350-423, CPU statement
 * e_natten/pytorch.py:228-288).  dK and dV are produced by gathering over each
 * key's inverse neighbourhood (pytorch.py:261-270), not by atomics, so results
 * are deterministic and the outputs need no zero-fill.
 *
 *   o, d_o      [B, heads, H, W, D] dtype (forward output, upstream gradient), read
 *               through o_strides / do_strides
 *   lse         as written by enatten2d_fwd with the same scale
 *   dq, dk, dv  [B, heads, H, W, D] dtype, contiguous, fully overwritten
 *   workspace   enatten2d_bwd_workspace_bytes() bytes of device memory for this call's
 *               shape, kernel_size and dtype
 */
int enatten2d_bwd(const void *q, const void *k, const void *v, const void *o,
                  const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                  void *workspace, int B, int heads, int H, int W, int D,
                  int kernel_size, int dtype, const int64_t *q_strides,
                  const int64_t *k_strides, const int64_t *v_strides,
                  const int64_t *o_strides, const int64_t *do_strides, float scale,
                  void *stream);

/*
 * enatten2d_bwd that writes dq, dk and dv into strided tensors: grad_strides gives the
 * element strides of all three on (batch, head, row, column), unit stride on the channels
 * (NULL: contiguous, i.e. enatten2d_bwd).  It has no counterpart in the reference (whose
 * gradients are zeros_like(Q), e_natten/triton.py:528-530); it is what lets a dilated call
 * write the gradients of a strided sub-grid straight into the full tensors.  Strides that
 * are no multiples of 8 elements run on the general kernels; head_dim 128 with kernel_size 5
 * and float32 then take the two-pass / general kernels (their fused and matrix-core
 * backward write contiguous gradients only).
 */
int enatten2d_bwd_into(const void *q, const void *k, const void *v, const void *o,
                       const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                       void *workspace, int B, int heads, int H, int W, int D,
                       int kernel_size, int dtype, const int64_t *q_strides,
                       const int64_t *k_strides, const int64_t *v_strides,
                       const int64_t *o_strides, const int64_t *do_strides,
                       const int64_t *grad_strides, float scale, void *stream);

/*
 * enatten2d_bwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments and results as enatten2d_bwd without
 * the workspace: the two float32 per query live in a device array that is part of
 * this library (8 MiB on every GPU the library runs on, held until the process ends),
 * so calls of at most ENATTEN_STATIC_BWD_MAX_QUERIES = B * heads * H * W queries are
 * served and larger ones return ENATTEN_EUNSUPPORTED.  float32 calls run the matrix-core
 * backward with the array as its P / dS buffers while B * heads * H * W * 2 * kernel_size^2
 * floats fit the array's 2^21, and the general kernels beyond that.  The call allocates and
 * frees nothing.  The stream's device must be the current device.  All calls on one GPU
 * share the one array: calls that may overlap there (different streams, different
 * threads) race; order them.
 * Under stream capture: make one call on the device OUTSIDE capture first.  The first call on
 * a device looks up the array's address (hipGetSymbolAddress, which may load the code object
 * that backs the array) and the first call of every kernel family asks the runtime for the
 * kernel's occupancy; neither is promised to be legal, or free of allocations, while a
 * stream is capturing.  Later calls of the same family only launch kernels.
 */
#define ENATTEN_STATIC_BWD_MAX_QUERIES (1 << 20)
int enatten2d_bwd_static(const void *q, const void *k, const void *v, const void *o,
                         const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                         int B, int heads, int H, int W, int D, int kernel_size, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *do_strides, float scale, void *stream);

/*
 * Rectangular and causal windows, relative position bias.  They have no counterpart in the reference, which has
 * one odd kernel_size for both axes and no causal mode (e_natten/triton.py:489,
 * e_natten/pytorch.py:7-11); they follow NATTEN's definitions and are for callers that
 * move over from it.  Each axis has its own extent, kernel_h rows by kernel_w columns.
 * On a causal axis a query at position i attends the keys [max(i - k + 1, 0), i]: the last
 * k positions up to and including its own, fewer at the start of the axis, and k may be
 * even there; on the other axes the window is the reference's
 * clamp(i - k/2, 0, L - k) with k odd.  The same conventions as enatten2d_fwd /
 * enatten2d_bwd otherwise; the workspace holds 16 bytes per query (two float32, or two
 * doubles for float64 tensors) and, with a bias, kernel_h * kernel_w float32 per query more
 * (enatten2d_bwd_window_workspace_bytes).  A 1D causal (sliding-window) attention over
 * [B, heads, T, D] is the call with H = 1, kernel_h = 1, causal_h = 0.
 *
 * rpb, NULL or a relative position bias [heads, 2 * kernel_h - 1, 2 * kernel_w - 1] of the
 * tensors' element type, contiguous: the logit of (query, key) gets entry
 * (key - query + kernel - 1) of each axis added after the scaling (NATTEN's rule; centred
 * axes only; not for float64 tensors).  The backward then writes the bias gradient to d_rpb,
 * float32 of the same shape, fully overwritten: the dK/dV pass leaves dS of every (query,
 * window position) in the workspace and one more kernel sums each entry's pairs in a fixed
 * order, so d_rpb is bit-reproducible like dq, dk and dv (no atomics anywhere).
 *
 * Square, non-causal calls without a bias are handed to the kernels behind enatten2d_fwd /
 * enatten2d_bwd; everything else runs on the general kernels.
 */
int enatten2d_fwd_window(const void *q, const void *k, const void *v, const void *rpb, void *o,
                         float *lse, int B, int heads, int H, int W, int D, int kernel_h,
                         int kernel_w, int causal_h, int causal_w, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides, float scale,
                         void *stream);
size_t enatten2d_bwd_window_workspace_bytes(int B, int heads, int H, int W, int kernel_h,
                                            int kernel_w, int with_rpb);
int enatten2d_bwd_window(const void *q, const void *k, const void *v, const void *rpb,
                         const void *o, const void *d_o, const float *lse, void *dq, void *dk,
                         void *dv, float *d_rpb, void *workspace, int B, int heads, int H, int W,
                         int D, int kernel_h, int kernel_w, int causal_h, int causal_w, int dtype,
                         const int64_t *q_strides, const int64_t *k_strides,
                         const int64_t *v_strides, const int64_t *o_strides,
                         const int64_t *do_strides, float scale, void *stream);

/*
 * 1D neighborhood attention on [B, heads, T, D] tensors: query t attends the
 * kernel_size keys starting at clamp(t - kernel_size/2, 0, T - kernel_size).
 * Replace the launches of _attn_fwd_1d / _attn_bwd_1d in Natten1d
 * (e_natten/triton.py:444-450, :472-481; CPU statement e_natten/pytorch.py:46-156).
 * Same conventions as the 2D calls; the stride arrays are int64_t[3] for the
 * (batch, head, position) axes, NULL for contiguous; lse is [B, heads, T].
 */
int enatten1d_fwd(const void *q, const void *k, const void *v, void *o, float *lse,
                  int B, int heads, int T, int D, int kernel_size, int dtype,
                  const int64_t *q_strides, const int64_t *k_strides,
                  const int64_t *v_strides, const int64_t *o_strides, float scale,
                  void *stream);
/* 16 bytes per position: two float32, or two doubles for float64 tensors (16-byte aligned) */
size_t enatten1d_bwd_workspace_bytes(int B, int heads, int T);
int enatten1d_bwd(const void *q, const void *k, const void *v, const void *o,
                  const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                  void *workspace, int B, int heads, int T, int D, int kernel_size,
                  int dtype, const int64_t *q_strides, const int64_t *k_strides,
                  const int64_t *v_strides, const int64_t *o_strides,
                  const int64_t *do_strides, float scale, void *stream);
/* enatten1d_bwd with dq, dk, dv written through grad_strides (batch, head, position), as
 * enatten2d_bwd_into */
int enatten1d_bwd_into(const void *q, const void *k, const void *v, const void *o,
                  const void *d_o, const float *lse, void *dq, void *dk, void *dv,
                  void *workspace, int B, int heads, int T, int D, int kernel_size,
                  int dtype, const int64_t *q_strides, const int64_t *k_strides,
                  const int64_t *v_strides, const int64_t *o_strides,
                  const int64_t *do_strides, const int64_t *grad_strides,
                       float scale, void *stream);

/*
 * Per-kernel timing aid for benchmarks (no counterpart in the reference, whose
 * bench.py:28,59 times whole calls with triton.testing.do_bench).  While
 * enabled, kernels this library launches are bracketed by HIP events on the
 * launch stream.  enatten_profile_enable(n), n >= 1, clears the figures and
 * times every n-th launch of each kernel (an event record costs a few
 * microseconds of queue time, so sampling keeps the timed loop undisturbed);
 * enatten_profile_enable(0) stops, waits for the recorded events, keeps their
 * durations and destroys them, so no HIP object is left behind; the return value
 * is the previous setting.  enatten_profile_read returns how many launches of one
 * kernel were timed and their summed duration (it also waits for and collects
 * what has been recorded so far).  At most 8192 launches per kernel are timed
 * between two enables.  Safe to call while other threads launch; while it is off
 * a launch reads one flag and nothing else.
 */
enum { ENATTEN_KERNEL_FWD = 0, ENATTEN_KERNEL_BWD_DQ = 1, ENATTEN_KERNEL_BWD_DKDV = 2,
       ENATTEN_KERNEL_BWD_FUSED = 3, ENATTEN_KERNEL_COUNT = 4 };
int enatten_profile_enable(int on);
int enatten_profile_read(int kernel, int *launches, double *total_ms);
/* What the brackets themselves added to total_ms: after each timed launch's closing
 * event a further event is recorded with nothing in between, and the time between
 * those two (the cost of one event on a busy queue, about 5 us on MI355X) is summed
 * here over the same launches.  total_ms minus this is the kernels' own time; without
 * the correction the brackets of one step add up to more than the step's wall time. */
int enatten_profile_read_overhead(int kernel, double *total_empty_ms);
/* Name of the device kernel last launched for that slot ("" if none yet). */
const char *enatten_profile_kernel_name(int kernel);

#ifdef __cplusplus
}
#endif
#endif /* ENATTEN_H */
