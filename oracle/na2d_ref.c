/*
 * CPU oracle for 2D neighborhood attention, plain C with OpenMP.
 *
 * TEST INFRASTRUCTURE ONLY: loaded by tests/, the smoke check and the
 * cpu_baseline leg of the benchmark.  The product library never links it.
 *
 * It restates the algorithm of the reference's e_natten/pytorch.py:
 *   window rule            pytorch.py:7-11   -> na2d_win_start
 *   inverse neighbourhood  pytorch.py:13-23  -> na2d_inv_range
 *   forward per query      pytorch.py:196-202 (S = q K_w^T, softmax, P V_w)
 *   dQ per query           pytorch.py:248-258 (dS = (diag P - P P^T) dP, dQ = dS K_w)
 *   dK, dV per key         pytorch.py:261-288 (gather over the inverse
 *                          neighbourhood; slot of the key inside the query's
 *                          window is (x - win_start(xi), y - win_start(yi)))
 * with one deliberate difference in schedule, not in result: each query's P
 * and dS are computed once and kept, instead of being recomputed for every
 * (key, query) pair as pytorch.py:271-281 does.
 *
 * Tensors are contiguous float32 [S][H][W][D] with S = batch*heads; all sums
 * are carried in double.  `scale` multiplies the logits (the reference uses
 * none, i.e. 1.0).
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int na2d_win_start(int i, int L, int k) {
    int s = i - k / 2;
    if (s < 0) s = 0;
    if (s > L - k) s = L - k;
    return s;
}

void na2d_inv_range(int i, int L, int k, int *lo, int *hi) {
    *lo = (i < k) ? 0 : i - k / 2;
    *hi = (i >= L - k) ? L : i + k / 2 + 1;
}

static void set_threads(int nthreads) {
#ifdef _OPENMP
    if (nthreads > 0) omp_set_num_threads(nthreads);
#else
    (void)nthreads;
#endif
}

int na2d_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* softmax probabilities of one query over its k*k window; returns log-sum-exp */
static double window_softmax(const float *qv, const float *kslab, int W, int D,
                             int x0, int y0, int kh, int kw, double scale, double *p) {
    double m = -INFINITY;
    for (int a = 0; a < kh; a++)
        for (int c = 0; c < kw; c++) {
            const float *kv = kslab + ((size_t)(x0 + a) * W + (y0 + c)) * D;
            double s = 0.0;
            for (int e = 0; e < D; e++) s += (double)qv[e] * (double)kv[e];
            s *= scale;
            p[a * kw + c] = s;
            if (s > m) m = s;
        }
    double z = 0.0;
    for (int j = 0; j < kh * kw; j++) { p[j] = exp(p[j] - m); z += p[j]; }
    for (int j = 0; j < kh * kw; j++) p[j] /= z;
    return m + log(z);
}

/* Rectangular kh x kw window; kh = 1 with H = 1 is the 1D operator of
 * pytorch.py:46-156 (same window rule along the one axis). */
void na2d_fwd_rect_f32(const float *q, const float *k, const float *v, float *o,
                       float *lse, int S, int H, int W, int D, int kh, int kw,
                       float scale, int nthreads) {
    set_threads(nthreads);
    const size_t slab = (size_t)H * W * D;
#pragma omp parallel
    {
        double *p = (double *)malloc(sizeof(double) * kh * kw);
        double *acc = (double *)malloc(sizeof(double) * D);
#pragma omp for collapse(2) schedule(static)
        for (int s = 0; s < S; s++)
            for (int x = 0; x < H; x++) {
                int x0 = na2d_win_start(x, H, kh);
                for (int y = 0; y < W; y++) {
                    int y0 = na2d_win_start(y, W, kw);
                    size_t qi = s * slab + ((size_t)x * W + y) * D;
                    double l = window_softmax(q + qi, k + s * slab, W, D, x0, y0, kh, kw, scale, p);
                    for (int e = 0; e < D; e++) acc[e] = 0.0;
                    for (int a = 0; a < kh; a++)
                        for (int c = 0; c < kw; c++) {
                            const float *vv = v + s * slab + ((size_t)(x0 + a) * W + (y0 + c)) * D;
                            double pj = p[a * kw + c];
                            for (int e = 0; e < D; e++) acc[e] += pj * (double)vv[e];
                        }
                    for (int e = 0; e < D; e++) o[qi + e] = (float)acc[e];
                    if (lse) lse[(size_t)s * H * W + (size_t)x * W + y] = (float)l;
                }
            }
        free(p);
        free(acc);
    }
}

void na2d_fwd_f32(const float *q, const float *k, const float *v, float *o,
                  float *lse, int S, int H, int W, int D, int ks, float scale,
                  int nthreads) {
    na2d_fwd_rect_f32(q, k, v, o, lse, S, H, W, D, ks, ks, scale, nthreads);
}

void na2d_bwd_rect_f32(const float *q, const float *k, const float *v, const float *d_o,
                       float *dq, float *dk, float *dv, int S, int H, int W, int D,
                       int kh, int kw, float scale, int nthreads) {
    set_threads(nthreads);
    const size_t slab = (size_t)H * W * D;
    const int kk = kh * kw;
    /* P and dS of every query, kept so the key-side gather can read them */
    double *P = (double *)malloc(sizeof(double) * (size_t)S * H * W * kk);
    double *dS = (double *)malloc(sizeof(double) * (size_t)S * H * W * kk);
#pragma omp parallel
    {
        double *dp = (double *)malloc(sizeof(double) * kk);
        double *acc = (double *)malloc(sizeof(double) * D);
        double *acc2 = (double *)malloc(sizeof(double) * D);
        /* query side: P, dS = (diag P - P P^T) dP, dQ = scale * dS K_w */
#pragma omp for collapse(2) schedule(static)
        for (int s = 0; s < S; s++)
            for (int x = 0; x < H; x++) {
                int x0 = na2d_win_start(x, H, kh);
                for (int y = 0; y < W; y++) {
                    int y0 = na2d_win_start(y, W, kw);
                    size_t tok = (size_t)s * H * W + (size_t)x * W + y;
                    size_t qi = s * slab + ((size_t)x * W + y) * D;
                    double *p = P + tok * kk, *ds = dS + tok * kk;
                    window_softmax(q + qi, k + s * slab, W, D, x0, y0, kh, kw, scale, p);
                    for (int a = 0; a < kh; a++)
                        for (int c = 0; c < kw; c++) {
                            const float *vv = v + s * slab + ((size_t)(x0 + a) * W + (y0 + c)) * D;
                            double t = 0.0;
                            for (int e = 0; e < D; e++) t += (double)d_o[qi + e] * (double)vv[e];
                            dp[a * kw + c] = t;
                        }
                    /* Jacobian row i: P_i (delta_ij - P_j) */
                    for (int i = 0; i < kk; i++) {
                        double t = 0.0;
                        for (int j = 0; j < kk; j++)
                            t += ((i == j ? p[i] : 0.0) - p[i] * p[j]) * dp[j];
                        ds[i] = t;
                    }
                    for (int e = 0; e < D; e++) acc[e] = 0.0;
                    for (int a = 0; a < kh; a++)
                        for (int c = 0; c < kw; c++) {
                            const float *kv = k + s * slab + ((size_t)(x0 + a) * W + (y0 + c)) * D;
                            double t = ds[a * kw + c];
                            for (int e = 0; e < D; e++) acc[e] += t * (double)kv[e];
                        }
                    for (int e = 0; e < D; e++) dq[qi + e] = (float)(acc[e] * scale);
                }
            }
        /* key side: gather over the inverse neighbourhood */
#pragma omp for collapse(2) schedule(static)
        for (int s = 0; s < S; s++)
            for (int x = 0; x < H; x++) {
                int qx0, qx1;
                na2d_inv_range(x, H, kh, &qx0, &qx1);
                for (int y = 0; y < W; y++) {
                    int qy0, qy1;
                    na2d_inv_range(y, W, kw, &qy0, &qy1);
                    for (int e = 0; e < D; e++) { acc[e] = 0.0; acc2[e] = 0.0; }
                    for (int xi = qx0; xi < qx1; xi++) {
                        int wx = na2d_win_start(xi, H, kh);
                        for (int yi = qy0; yi < qy1; yi++) {
                            int wy = na2d_win_start(yi, W, kw);
                            int slot = (x - wx) * kw + (y - wy);
                            size_t tok = (size_t)s * H * W + (size_t)xi * W + yi;
                            size_t qi = s * slab + ((size_t)xi * W + yi) * D;
                            double a = dS[tok * kk + slot], b = P[tok * kk + slot];
                            for (int e = 0; e < D; e++) {
                                acc[e] += a * (double)q[qi + e];
                                acc2[e] += b * (double)d_o[qi + e];
                            }
                        }
                    }
                    size_t ki = s * slab + ((size_t)x * W + y) * D;
                    for (int e = 0; e < D; e++) {
                        dk[ki + e] = (float)(acc[e] * scale);
                        dv[ki + e] = (float)acc2[e];
                    }
                }
            }
        free(dp);
        free(acc);
        free(acc2);
    }
    free(P);
    free(dS);
}

void na2d_bwd_f32(const float *q, const float *k, const float *v, const float *d_o,
                  float *dq, float *dk, float *dv, int S, int H, int W, int D,
                  int ks, float scale, int nthreads) {
    na2d_bwd_rect_f32(q, k, v, d_o, dq, dk, dv, S, H, W, D, ks, ks, scale, nthreads);
}
