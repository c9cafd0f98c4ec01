/*
 * TEST INFRASTRUCTURE ONLY -- CPU oracle for the SS2D inference hot path.
 *
 * This file restates, in plain C, the arithmetic of three operators of
 * MzeroMiko/VMamba.  It is the checker the HIP kernels are compared against;
 * nothing in the shipped package links, loads or calls it.
 *
 *   ss2d_oracle_cross_scan      <- classification/models/csm_triton.py:22-29
 *                                  (cross_scan_fwd, scans=0, channel-first)
 *   ss2d_oracle_cross_merge_*   <- classification/models/csm_triton.py:56-62
 *                                  (cross_merge_fwd, scans=0, channel-first;
 *                                  add order (y0+flip y2) + T(y1+flip y3)),
 *                                  alternative left-to-right order of the
 *                                  Triton kernel: csm_triton.py:362-370
 *   ss2d_oracle_selective_scan  <- kernels/selective_scan/test_selective_scan.py:168-234
 *                                  (selective_scan_ref) == classification/models/csms6s.py:25-68
 *                                  with the kernel-level conventions of
 *                                  .../cusoflex/selective_scan_fwd_kernel_oflex.cuh:88-177
 *                                  (group ids :90-91, softplus threshold :126,
 *                                  chunk-end state x :164-167) and
 *                                  .../cusoflex/selective_scan_oflex.cpp:206-208
 *                                  (2048-element chunks, x layout).
 *
 * Pinned by tests/test_oracle_*.py: hand-derived known answers, closed forms
 * (geometric series, cumsum reduction, L=1), a float64 brute force, the
 * second formulation with library transpose/flip, adjointness and
 * permutation invariants.  No function here is "parity unpinned".
 *
 * All tensors are dense row-major ("contiguous") unless a stride is given.
 * bf16 values travel as uint16_t bit patterns.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define SS2D_ORACLE_CHUNK 2048 /* selective_scan_oflex.cpp:206 */

int ss2d_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ---- bf16 <-> f32, round-to-nearest-even (what torch does on CPU) -------- */
static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}
void ss2d_oracle_bf16_to_f32(const uint16_t *src, float *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}
void ss2d_oracle_f32_to_bf16(const float *src, uint16_t *dst, int64_t n) {
    for (int64_t i = 0; i < n; ++i) dst[i] = f32_to_bf16(src[i]);
}

/* ---- CrossScan ------------------------------------------------------------
 * x (B,C,H,W) -> y (B,4,C,L), L=H*W, any element size, pure permutation:
 *   y[b,0,c,h*W+w]       = x[b,c,h,w]            row-major
 *   y[b,1,c,w*H+h]       = x[b,c,h,w]            column-major (transpose)
 *   y[b,2,c,L-1-(h*W+w)] = x[b,c,h,w]            reversed row-major
 *   y[b,3,c,L-1-(w*H+h)] = x[b,c,h,w]            reversed column-major
 */
int ss2d_oracle_cross_scan(const void *x_, void *y_, int B, int C, int H, int W, int elem_bytes) {
    if (B < 0 || C < 0 || H < 0 || W < 0 || elem_bytes <= 0) return -1;
    const char *x = (const char *)x_;
    char *y = (char *)y_;
    const int64_t L = (int64_t)H * W;
    const int64_t maps = (int64_t)B * C;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < maps; ++m) {
        const int64_t b = m / C, c = m % C;
        const char *xm = x + m * L * elem_bytes;
        char *y0 = y + ((b * 4 + 0) * C + c) * L * elem_bytes;
        char *y1 = y + ((b * 4 + 1) * C + c) * L * elem_bytes;
        char *y2 = y + ((b * 4 + 2) * C + c) * L * elem_bytes;
        char *y3 = y + ((b * 4 + 3) * C + c) * L * elem_bytes;
        for (int h = 0; h < H; ++h)
            for (int w = 0; w < W; ++w) {
                const int64_t r = (int64_t)h * W + w, t = (int64_t)w * H + h;
                const char *s = xm + r * elem_bytes;
                memcpy(y0 + r * elem_bytes, s, elem_bytes);
                memcpy(y1 + t * elem_bytes, s, elem_bytes);
                memcpy(y2 + (L - 1 - r) * elem_bytes, s, elem_bytes);
                memcpy(y3 + (L - 1 - t) * elem_bytes, s, elem_bytes);
            }
    }
    return 0;
}

/* ---- CrossMerge -----------------------------------------------------------
 * ys (B,4,C,L) -> out (B,C,L).  With r=h*W+w and t=w*H+h:
 *   order 0 (torch):  out[r] = (y0[r] + y2[L-1-r]) + (y1[t] + y3[L-1-t])
 *   order 1 (Triton): out[r] = ((y0[r] + y1[t]) + y2[L-1-r]) + y3[L-1-t]
 * Every pairwise add is rounded to the tensor dtype, as elementwise torch ops do.
 */
int ss2d_oracle_cross_merge_f32(const float *ys, float *out, int B, int C, int H, int W, int order) {
    if (order != 0 && order != 1) return -1;
    const int64_t L = (int64_t)H * W, maps = (int64_t)B * C;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < maps; ++m) {
        const int64_t b = m / C, c = m % C;
        const float *y0 = ys + ((b * 4 + 0) * C + c) * L, *y1 = ys + ((b * 4 + 1) * C + c) * L;
        const float *y2 = ys + ((b * 4 + 2) * C + c) * L, *y3 = ys + ((b * 4 + 3) * C + c) * L;
        float *o = out + m * L;
        for (int h = 0; h < H; ++h)
            for (int w = 0; w < W; ++w) {
                const int64_t r = (int64_t)h * W + w, t = (int64_t)w * H + h;
                if (order == 0) {
                    volatile float s02 = y0[r] + y2[L - 1 - r];
                    volatile float s13 = y1[t] + y3[L - 1 - t];
                    o[r] = s02 + s13;
                } else {
                    volatile float s = y0[r] + y1[t];
                    s = s + y2[L - 1 - r];
                    o[r] = s + y3[L - 1 - t];
                }
            }
    }
    return 0;
}

int ss2d_oracle_cross_merge_bf16(const uint16_t *ys, uint16_t *out, int B, int C, int H, int W, int order) {
    if (order != 0 && order != 1) return -1;
    const int64_t L = (int64_t)H * W, maps = (int64_t)B * C;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < maps; ++m) {
        const int64_t b = m / C, c = m % C;
        const uint16_t *y0 = ys + ((b * 4 + 0) * C + c) * L, *y1 = ys + ((b * 4 + 1) * C + c) * L;
        const uint16_t *y2 = ys + ((b * 4 + 2) * C + c) * L, *y3 = ys + ((b * 4 + 3) * C + c) * L;
        uint16_t *o = out + m * L;
        for (int h = 0; h < H; ++h)
            for (int w = 0; w < W; ++w) {
                const int64_t r = (int64_t)h * W + w, t = (int64_t)w * H + h;
                if (order == 0) {
                    uint16_t s02 = f32_to_bf16(bf16_to_f32(y0[r]) + bf16_to_f32(y2[L - 1 - r]));
                    uint16_t s13 = f32_to_bf16(bf16_to_f32(y1[t]) + bf16_to_f32(y3[L - 1 - t]));
                    o[r] = f32_to_bf16(bf16_to_f32(s02) + bf16_to_f32(s13));
                } else {
                    uint16_t s = f32_to_bf16(bf16_to_f32(y0[r]) + bf16_to_f32(y1[t]));
                    s = f32_to_bf16(bf16_to_f32(s) + bf16_to_f32(y2[L - 1 - r]));
                    o[r] = f32_to_bf16(bf16_to_f32(s) + bf16_to_f32(y3[L - 1 - t]));
                }
            }
    }
    return 0;
}

/* ---- Selective scan forward -------------------------------------------------
 * Inputs are fp32 (callers widen bf16/f16 exactly):
 *   u      (batch, dim, L)
 *   delta  (batch, delta_dim, L)   dim % delta_dim == 0; channel d uses row d/(dim/delta_dim)
 *   A      (dim, N)
 *   Bm,Cm  (batch, G, N, L)        dim % G == 0; channel d uses group d/(dim/G)
 *   D      (dim) or NULL, delta_bias (delta_dim) or NULL
 * Recurrence per (b,d), all in fp32 (or fp64 when wide != 0):
 *   dl   = delta + bias;  if softplus: dl = dl > 20 ? dl : log1p(exp(dl))
 *   h_n  = exp(dl*A[d,n]) * h_n + dl*B[n,t]*u
 *   y_t  = sum_n h_n*C[n,t] + D[d]*u
 * Outputs:
 *   out  (batch, dim, L) fp32 (may be NULL)
 *   xst  (batch, dim, n_chunks, 2N) fp32 or NULL: after every 2048-element
 *        chunk, xst[..,2n] = running product of a since t=0, xst[..,2n+1] = h_n
 *   out64 (batch, dim, L) double, only written when wide != 0 (may be NULL)
 */
int ss2d_oracle_selective_scan(const float *u, const float *delta, const float *A, const float *Bm,
                               const float *Cm, const float *D, const float *delta_bias,
                               int delta_softplus, int batch, int dim, int L, int N, int G,
                               int delta_dim, float *out, float *xst, double *out64, int wide) {
    if (batch < 0 || dim <= 0 || L < 0 || N <= 0 || G <= 0 || delta_dim <= 0) return -1;
    if (dim % G != 0 || dim % delta_dim != 0) return -2;
    const int n_chunks = (L + SS2D_ORACLE_CHUNK - 1) / SS2D_ORACLE_CHUNK;
    const int dpg = dim / G, dpd = dim / delta_dim;
    const int64_t rows = (int64_t)batch * dim;
    int fail = 0;
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t r = 0; r < rows; ++r) {
        const int64_t b = r / dim;
        const int d = (int)(r % dim);
        const int g = d / dpg, dg = d / dpd;
        const float *ur = u + r * L;
        const float *dr = delta + (b * delta_dim + dg) * L;
        const float *Br = Bm + (b * G + g) * (int64_t)N * L;
        const float *Cr = Cm + (b * G + g) * (int64_t)N * L;
        const float Dv = D ? D[d] : 0.0f;
        const float bias = delta_bias ? delta_bias[dg] : 0.0f;
        if (!wide) {
            float *h = (float *)calloc((size_t)N, sizeof(float));
            float *ap = (float *)malloc((size_t)N * sizeof(float));
            if (!h || !ap) { fail = 1; free(h); free(ap); continue; }
            for (int n = 0; n < N; ++n) ap[n] = 1.0f;
            for (int t = 0; t < L; ++t) {
                float dl = dr[t] + bias;
                if (delta_softplus) dl = dl > 20.0f ? dl : log1pf(expf(dl));
                const float uv = ur[t];
                float y = 0.0f;
                for (int n = 0; n < N; ++n) {
                    const float a = expf(dl * A[(int64_t)d * N + n]);
                    const float bu = dl * Br[(int64_t)n * L + t] * uv;
                    h[n] = a * h[n] + bu;
                    ap[n] *= a;
                    y += h[n] * Cr[(int64_t)n * L + t];
                }
                if (out) out[r * L + t] = y + uv * Dv;
                if (xst && ((t + 1) % SS2D_ORACLE_CHUNK == 0 || t == L - 1)) {
                    float *xs = xst + (r * n_chunks + t / SS2D_ORACLE_CHUNK) * 2 * (int64_t)N;
                    for (int n = 0; n < N; ++n) { xs[2 * n] = ap[n]; xs[2 * n + 1] = h[n]; }
                }
            }
            free(h); free(ap);
        } else {
            double *h = (double *)calloc((size_t)N, sizeof(double));
            if (!h) { fail = 1; continue; }
            for (int t = 0; t < L; ++t) {
                double dl = (double)dr[t] + (double)bias;
                if (delta_softplus) dl = dl > 20.0 ? dl : log1p(exp(dl));
                const double uv = ur[t];
                double y = 0.0;
                for (int n = 0; n < N; ++n) {
                    const double a = exp(dl * (double)A[(int64_t)d * N + n]);
                    h[n] = a * h[n] + dl * (double)Br[(int64_t)n * L + t] * uv;
                    y += h[n] * (double)Cr[(int64_t)n * L + t];
                }
                if (out64) out64[r * L + t] = y + uv * (double)Dv;
            }
            free(h);
        }
    }
    return fail ? -3 : 0;
}
