/*
 * CPU oracle for the FastConv convolution hot path (see fastconv_oracle.h).
 * TEST INFRASTRUCTURE ONLY: never linked into or called by the shipped
 * library.  Plain C, OpenMP over independent outputs only (the summation
 * order inside one output element is the reference's).
 */
#include "fastconv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

int fco_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* conv_layer.h:68-69: out = (in + pad_a + pad_b - k) / stride + 1 */
int fco_out_h(const fco_shape *s) { return (s->H + s->pt + s->pb - s->kh) / s->sh + 1; }
int fco_out_w(const fco_shape *s) { return (s->W + s->pl + s->pr - s->kw) / s->sw + 1; }

static int shape_ok(const fco_shape *s) {
    if (s->N <= 0 || s->C <= 0 || s->H <= 0 || s->W <= 0 || s->K <= 0) return 0;
    if (s->kh <= 0 || s->kw <= 0 || s->sh <= 0 || s->sw <= 0) return 0;
    if (s->pt < 0 || s->pb < 0 || s->pl < 0 || s->pr < 0) return 0;
    if (s->H + s->pt + s->pb < s->kh || s->W + s->pl + s->pr < s->kw) return 0;
    return 1;
}

/*
 * Direct convolution, fp32 accumulation.
 * convLayer/naiveConv_wudu.h:48-81: for each output channel and output pixel,
 * for each input channel a partial `total` is summed over (kh, kw) in row-major
 * tap order skipping out-of-image taps, and `sum += total` over channels; the
 * bias is added last.  convLayer/naiveConv.h:24-64 is the 3x3 / stride-1
 * special case of the same loop nest (out-of-image taps add value 0 instead of
 * being skipped, which is the same number).
 */
int fco_naive_conv_f32(const fco_shape *s, const float *x, const float *w,
                       const float *bias, int bias_mode, float *y) {
    if (!shape_ok(s)) return -1;
    const int OH = fco_out_h(s), OW = fco_out_w(s);
    const long in_page = (long)s->H * s->W, out_page = (long)OH * OW;
    const int kpage = s->kh * s->kw;
    const long krow = (long)s->C * kpage;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < s->N; n++) {
        for (int oc = 0; oc < s->K; oc++) {
            const float *xn = x + (long)n * s->C * in_page;
            float *yo = y + ((long)n * s->K + oc) * out_page;
            for (long pix = 0; pix < out_page; pix++) {
                const int h0 = (int)(pix / OW) * s->sh - s->pt;
                const int w0 = (int)(pix % OW) * s->sw - s->pl;
                float sum = 0.f;
                for (int ic = 0; ic < s->C; ic++) {
                    const float *ip = xn + ic * in_page;
                    const float *kp = w + oc * krow + (long)ic * kpage;
                    float total = 0.f;
                    for (int i = 0; i < s->kh; i++) {
                        for (int j = 0; j < s->kw; j++) {
                            const int hh = h0 + i, ww = w0 + j;
                            if (hh < 0 || hh >= s->H || ww < 0 || ww >= s->W) continue;
                            total += ip[(long)hh * s->W + ww] * kp[i * s->kw + j];
                        }
                    }
                    sum += total;
                }
                if (bias_mode == 1) sum += bias[oc];
                else if (bias_mode == 2) sum += bias[oc * out_page + pix];
                yo[pix] = sum;
            }
        }
    }
    return 0;
}

/* Same loop nest with every product and sum in double: the "truth" the error
 * metrics are quoted against. */
int fco_naive_conv_f64(const fco_shape *s, const float *x, const float *w,
                       const float *bias, int bias_mode, double *y) {
    if (!shape_ok(s)) return -1;
    const int OH = fco_out_h(s), OW = fco_out_w(s);
    const long in_page = (long)s->H * s->W, out_page = (long)OH * OW;
    const int kpage = s->kh * s->kw;
    const long krow = (long)s->C * kpage;
#pragma omp parallel for collapse(2) schedule(static)
    for (int n = 0; n < s->N; n++) {
        for (int oc = 0; oc < s->K; oc++) {
            const float *xn = x + (long)n * s->C * in_page;
            double *yo = y + ((long)n * s->K + oc) * out_page;
            for (long pix = 0; pix < out_page; pix++) {
                const int h0 = (int)(pix / OW) * s->sh - s->pt;
                const int w0 = (int)(pix % OW) * s->sw - s->pl;
                double sum = 0.0;
                for (int ic = 0; ic < s->C; ic++) {
                    const float *ip = xn + ic * in_page;
                    const float *kp = w + oc * krow + (long)ic * kpage;
                    for (int i = 0; i < s->kh; i++) {
                        for (int j = 0; j < s->kw; j++) {
                            const int hh = h0 + i, ww = w0 + j;
                            if (hh < 0 || hh >= s->H || ww < 0 || ww >= s->W) continue;
                            sum += (double)ip[(long)hh * s->W + ww] * (double)kp[i * s->kw + j];
                        }
                    }
                }
                if (bias_mode == 1) sum += (double)bias[oc];
                else if (bias_mode == 2) sum += (double)bias[oc * out_page + pix];
                yo[pix] = sum;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Winograd F(6x6, 3x3)                                                      */
/* ------------------------------------------------------------------------ */

/* B^T: the linear map winoF63ZC/winoF63ZC.cpp:137-166 (input_transform_v1)
 * applies to 8 samples, written out as a matrix. */
static const float kBT[8][8] = {
    {1.f, 0.f, -5.25f, 0.f, 5.25f, 0.f, -1.f, 0.f},
    {0.f, 1.f, 1.f, -4.25f, -4.25f, 1.f, 1.f, 0.f},
    {0.f, -1.f, 1.f, 4.25f, -4.25f, -1.f, 1.f, 0.f},
    {0.f, 0.5f, 0.25f, -2.5f, -1.25f, 2.f, 1.f, 0.f},
    {0.f, -0.5f, 0.25f, 2.5f, -1.25f, -2.f, 1.f, 0.f},
    {0.f, 2.f, 4.f, -2.5f, -5.f, 0.5f, 1.f, 0.f},
    {0.f, -2.f, 4.f, 2.5f, -5.f, -0.5f, 1.f, 0.f},
    {0.f, -1.f, 0.f, 5.25f, 0.f, -5.25f, 0.f, 1.f},
};

/* G: winoF63ZC/winoF63ZC.cpp:28-78 (winograd_f6k3_kernel_transform_v1),
 * rows scaled by 1, -2/9, -2/9, 1/90, 1/90, 1/180, 1/180, 1. */
static const double kGd[8][3] = {
    {1.0, 0.0, 0.0},
    {-2.0 / 9, -2.0 / 9, -2.0 / 9},
    {-2.0 / 9, 2.0 / 9, -2.0 / 9},
    {1.0 / 90, 2.0 / 90, 4.0 / 90},
    {1.0 / 90, -2.0 / 90, 4.0 / 90},
    {4.0 / 180, 2.0 / 180, 1.0 / 180},
    {4.0 / 180, -2.0 / 180, 1.0 / 180},
    {0.0, 0.0, 1.0},
};

/* A^T: winoF63ZC/winoF63ZC.cpp:181-228
 * (winograd_f6k3_output_transform_inplace_v1). */
static const float kAT[6][8] = {
    {1.f, 1.f, 1.f, 1.f, 1.f, 32.f, 32.f, 0.f},
    {0.f, 1.f, -1.f, 2.f, -2.f, 16.f, -16.f, 0.f},
    {0.f, 1.f, 1.f, 4.f, 4.f, 8.f, 8.f, 0.f},
    {0.f, 1.f, -1.f, 8.f, -8.f, 4.f, -4.f, 0.f},
    {0.f, 1.f, 1.f, 16.f, 16.f, 2.f, 2.f, 0.f},
    {0.f, 1.f, -1.f, 32.f, -32.f, 1.f, -1.f, 1.f},
};

void fco_wino_matrices(float BT[64], float G[24], float AT[48]) {
    for (int i = 0; i < 8; i++)
        for (int j = 0; j < 8; j++) BT[i * 8 + j] = kBT[i][j];
    for (int i = 0; i < 8; i++)
        for (int j = 0; j < 3; j++) G[i * 3 + j] = (float)kGd[i][j];
    for (int i = 0; i < 6; i++)
        for (int j = 0; j < 8; j++) AT[i * 8 + j] = kAT[i][j];
}

/* winoF63ZC/winoF63ZC.cpp:336-338: tileH = (OH+5)/6, tileW = (OW+5)/6 */
int fco_wino_tiles_h(const fco_shape *s) { return (fco_out_h(s) + 5) / 6; }
int fco_wino_tiles_w(const fco_shape *s) { return (fco_out_w(s) + 5) / 6; }

static int wino_shape_ok(const fco_shape *s) {
    return shape_ok(s) && s->kh == 3 && s->kw == 3 && s->sh == 1 && s->sw == 1;
}

/* U = G g G^T per (k, c); winoF63ZC/winoF63ZC.cpp:433-500 applies the 1-D
 * kernel transform, transposes, and applies it again. */
int fco_wino_filter_transform(const float *w, float *U, int K, int C) {
    if (K <= 0 || C <= 0) return -1;
    const long KC = (long)K * C;
#pragma omp parallel for schedule(static)
    for (long kc = 0; kc < KC; kc++) {
        const float *g = w + kc * 9;
        float tmp[8][3];
        for (int i = 0; i < 8; i++)
            for (int j = 0; j < 3; j++) {
                float a = 0.f;
                for (int r = 0; r < 3; r++) a += (float)kGd[i][r] * g[r * 3 + j];
                tmp[i][j] = a;
            }
        for (int i = 0; i < 8; i++)
            for (int j = 0; j < 8; j++) {
                float a = 0.f;
                for (int r = 0; r < 3; r++) a += tmp[i][r] * (float)kGd[j][r];
                U[(long)(i * 8 + j) * KC + kc] = a;
            }
    }
    return 0;
}

/* V = B^T d B per (c, tile).  Tile origin and zero fill:
 * winoF63ZC/winoF63ZC.cpp:543-544 (origin = 6*tile index - pad) and :574-612
 * (samples outside the image read as 0). */
int fco_wino_input_transform(const fco_shape *s, const float *x, float *V) {
    if (!wino_shape_ok(s)) return -1;
    const int tH = fco_wino_tiles_h(s), tW = fco_wino_tiles_w(s);
    const long tileN = (long)tH * tW, T = tileN * s->N;
    const long page = (long)s->H * s->W;
    const long CT = (long)s->C * T;
#pragma omp parallel for collapse(2) schedule(static)
    for (int c = 0; c < s->C; c++) {
        for (long t = 0; t < T; t++) {
            const int n = (int)(t / tileN);
            const int r = (int)(t % tileN);
            const int h0 = (r / tW) * 6 - s->pt, w0 = (r % tW) * 6 - s->pl;
            const float *ip = x + ((long)n * s->C + c) * page;
            float d[8][8], tmp[8][8];
            for (int i = 0; i < 8; i++)
                for (int j = 0; j < 8; j++) {
                    const int hh = h0 + i, ww = w0 + j;
                    d[i][j] = (hh >= 0 && hh < s->H && ww >= 0 && ww < s->W)
                                  ? ip[(long)hh * s->W + ww] : 0.f;
                }
            for (int i = 0; i < 8; i++)
                for (int j = 0; j < 8; j++) {
                    float a = 0.f;
                    for (int q = 0; q < 8; q++) a += kBT[i][q] * d[q][j];
                    tmp[i][j] = a;
                }
            for (int i = 0; i < 8; i++)
                for (int j = 0; j < 8; j++) {
                    float a = 0.f;
                    for (int q = 0; q < 8; q++) a += tmp[i][q] * kBT[j][q];
                    V[(long)(i * 8 + j) * CT + (long)c * T + t] = a;
                }
        }
    }
    return 0;
}

/* M[f][k][t] = sum_c U[f][k][c] V[f][c][t], channels summed in ascending
 * order.  winoF63ZC/TensorGEMMZC.cpp:443-583 computes the same contraction for
 * a 4x4 register block of (k, t) and 4 frequencies at a time. */
int fco_wino_gemm(const float *U, const float *V, float *M, int K, int C, long T) {
    if (K <= 0 || C <= 0 || T <= 0) return -1;
#pragma omp parallel for collapse(2) schedule(static)
    for (int f = 0; f < 64; f++) {
        for (int k = 0; k < K; k++) {
            float *m = M + ((long)f * K + k) * T;
            for (long t = 0; t < T; t++) m[t] = 0.f;
            for (int c = 0; c < C; c++) {
                const float u = U[((long)f * K + k) * C + c];
                const float *v = V + ((long)f * C + c) * T;
                for (long t = 0; t < T; t++) m[t] += u * v[t];
            }
        }
    }
    return 0;
}

/* Y = A^T m A per (k, tile), clipped to the image:
 * winoF63ZC/winoF63ZC.cpp:869-973 (edge clipping :924-969). */
int fco_wino_output_transform(const fco_shape *s, const float *M,
                              const float *bias, float *y) {
    if (!wino_shape_ok(s)) return -1;
    const int OH = fco_out_h(s), OW = fco_out_w(s);
    const int tH = fco_wino_tiles_h(s), tW = fco_wino_tiles_w(s);
    const long tileN = (long)tH * tW, T = tileN * s->N;
    const long KT = (long)s->K * T;
#pragma omp parallel for collapse(2) schedule(static)
    for (int k = 0; k < s->K; k++) {
        for (long t = 0; t < T; t++) {
            const int n = (int)(t / tileN);
            const int r = (int)(t % tileN);
            const int oh0 = (r / tW) * 6, ow0 = (r % tW) * 6;
            float m[8][8], tmp[6][8];
            for (int f = 0; f < 64; f++) m[f / 8][f % 8] = M[(long)f * KT + (long)k * T + t];
            for (int i = 0; i < 6; i++)
                for (int j = 0; j < 8; j++) {
                    float a = 0.f;
                    for (int q = 0; q < 8; q++) a += kAT[i][q] * m[q][j];
                    tmp[i][j] = a;
                }
            float *yo = y + ((long)n * s->K + k) * OH * OW;
            for (int i = 0; i < 6 && oh0 + i < OH; i++)
                for (int j = 0; j < 6 && ow0 + j < OW; j++) {
                    float a = 0.f;
                    for (int q = 0; q < 8; q++) a += tmp[i][q] * kAT[j][q];
                    if (bias) a += bias[k];
                    yo[(long)(oh0 + i) * OW + ow0 + j] = a;
                }
        }
    }
    return 0;
}

int fco_wino_conv_f32(const fco_shape *s, const float *x, const float *w,
                      const float *bias, float *y) {
    if (!wino_shape_ok(s)) return -1;
    const long T = (long)s->N * fco_wino_tiles_h(s) * fco_wino_tiles_w(s);
    float *U = (float *)malloc(sizeof(float) * 64 * (size_t)s->K * s->C);
    float *V = (float *)malloc(sizeof(float) * 64 * (size_t)s->C * T);
    float *M = (float *)malloc(sizeof(float) * 64 * (size_t)s->K * T);
    int rc = -2;
    if (U && V && M) {
        rc = fco_wino_filter_transform(w, U, s->K, s->C);
        if (!rc) rc = fco_wino_input_transform(s, x, V);
        if (!rc) rc = fco_wino_gemm(U, V, M, s->K, s->C, T);
        if (!rc) rc = fco_wino_output_transform(s, M, bias, y);
    }
    free(U); free(V); free(M);
    return rc;
}

/* ------------------------------------------------------------------------ */
/* im2col + GEMM                                                             */
/* ------------------------------------------------------------------------ */

/* Column matrix [C*kh*kw][N*OH*OW]; row (c,u,v), column (n,i,j) holds
 * x[n][c][u - pt + i*sh][v - pl + j*sw] or 0 outside the image:
 * convLayer/im2colConv.cpp:285-309. */
int fco_im2col(const fco_shape *s, const float *x, float *col) {
    if (!shape_ok(s)) return -1;
    const int OH = fco_out_h(s), OW = fco_out_w(s);
    const long ncols = (long)s->N * OH * OW;
    const int rows = s->C * s->kh * s->kw;
#pragma omp parallel for schedule(static)
    for (int row = 0; row < rows; row++) {
        const int c = row / (s->kh * s->kw);
        const int u = (row / s->kw) % s->kh, v = row % s->kw;
        float *dst = col + (long)row * ncols;
        for (int n = 0; n < s->N; n++) {
            const float *ip = x + ((long)n * s->C + c) * s->H * s->W;
            for (int i = 0; i < OH; i++)
                for (int j = 0; j < OW; j++) {
                    const int hh = u - s->pt + i * s->sh, ww = v - s->pl + j * s->sw;
                    *dst++ = (hh < 0 || hh >= s->H || ww < 0 || ww >= s->W)
                                 ? 0.f : ip[(long)hh * s->W + ww];
                }
        }
    }
    return 0;
}

/* C[M][Ncols] = A[M][Kred] * B[Kred][Ncols], reduction in ascending order
 * (the product convLayer/im2colConv.cpp:400-432 forms, on a zeroed C). */
void fco_sgemm(int M, long Ncols, int Kred, const float *A, const float *B, float *Cmat) {
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; m++) {
        float *c = Cmat + (long)m * Ncols;
        for (long j = 0; j < Ncols; j++) c[j] = 0.f;
        for (int k = 0; k < Kred; k++) {
            const float a = A[(long)m * Kred + k];
            const float *b = B + (long)k * Ncols;
            for (long j = 0; j < Ncols; j++) c[j] += a * b[j];
        }
    }
}

/* convLayer/im2colConv.h:23-25: M = K_out, N = OH*OW, K = C*kh*kw. */
int fco_im2col_conv_f32(const fco_shape *s, const float *x, const float *w,
                        const float *bias, float *y) {
    if (!shape_ok(s)) return -1;
    const int OH = fco_out_h(s), OW = fco_out_w(s);
    const long page = (long)OH * OW, ncols = (long)s->N * page;
    const int kred = s->C * s->kh * s->kw;
    float *col = (float *)malloc(sizeof(float) * (size_t)kred * ncols);
    float *out = (float *)malloc(sizeof(float) * (size_t)s->K * ncols);
    if (!col || !out) { free(col); free(out); return -2; }
    fco_im2col(s, x, col);
    fco_sgemm(s->K, ncols, kred, w, col, out);
    for (int n = 0; n < s->N; n++)
        for (int k = 0; k < s->K; k++)
            for (long p = 0; p < page; p++)
                y[((long)n * s->K + k) * page + p] =
                    out[(long)k * ncols + (long)n * page + p] + (bias ? bias[k] : 0.f);
    free(col); free(out);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* error metrics                                                             */
/* ------------------------------------------------------------------------ */

/* utility/helper.cpp:74-89: mean of |a-b| over the elements where it exceeds
 * 1e-5 (0 if there are none). */
float fco_diff_legacy(const float *a, const float *b, long len) {
    long num = 0;
    double dif = 0.0;
    for (long i = 0; i < len; i++) {
        const float err = fabsf(a[i] - b[i]);
        if (err > 1e-5f) { dif += err; num++; }
    }
    return num == 0 ? 0.f : (float)(dif / num);
}

double fco_max_rel_err_f32(const float *y, const double *ref, long len) {
    double maxerr = 0.0, maxref = 0.0;
    for (long i = 0; i < len; i++) {
        const double e = fabs((double)y[i] - ref[i]);
        if (!(e <= maxerr)) maxerr = e;            /* NaN propagates */
        if (fabs(ref[i]) > maxref) maxref = fabs(ref[i]);
    }
    return maxref > 0.0 ? maxerr / maxref : maxerr;
}

double fco_max_rel_err_f32f32(const float *y, const float *ref, long len) {
    double maxerr = 0.0, maxref = 0.0;
    for (long i = 0; i < len; i++) {
        const double e = fabs((double)y[i] - (double)ref[i]);
        if (!(e <= maxerr)) maxerr = e;
        if (fabs((double)ref[i]) > maxref) maxref = fabs((double)ref[i]);
    }
    return maxref > 0.0 ? maxerr / maxref : maxerr;
}

/* ------------------------------------------------------------------------ */
/* deterministic inputs                                                      */
/* ------------------------------------------------------------------------ */

static inline uint64_t rotl64(uint64_t v, int k) { return (v << k) | (v >> (64 - k)); }

typedef struct { uint64_t s[4]; } xo_state;

static uint64_t splitmix64_next(uint64_t *st) {
    uint64_t z = (*st += 0x9e3779b97f4a7c15ULL);
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
    return z ^ (z >> 31);
}

static void xo_seed(xo_state *x, uint64_t seed) {
    uint64_t sm = seed;
    for (int i = 0; i < 4; i++) x->s[i] = splitmix64_next(&sm);
}

static uint64_t xo_next(xo_state *x) {
    const uint64_t result = rotl64(x->s[1] * 5, 7) * 9;
    const uint64_t t = x->s[1] << 17;
    x->s[2] ^= x->s[0];
    x->s[3] ^= x->s[1];
    x->s[1] ^= x->s[2];
    x->s[0] ^= x->s[3];
    x->s[2] ^= t;
    x->s[3] = rotl64(x->s[3], 45);
    return result;
}

static double xo_unit(xo_state *x) { return (double)(xo_next(x) >> 11) * (1.0 / 9007199254740992.0); }

void fco_rng_raw(uint64_t seed, uint64_t *out, long n) {
    xo_state st; xo_seed(&st, seed);
    for (long i = 0; i < n; i++) out[i] = xo_next(&st);
}

void fco_rng_uniform(uint64_t seed, float lo, float hi, float *out, long n) {
    xo_state st; xo_seed(&st, seed);
    for (long i = 0; i < n; i++) out[i] = (float)((double)lo + ((double)hi - (double)lo) * xo_unit(&st));
}

void fco_rng_normal(uint64_t seed, float sigma, float *out, long n) {
    xo_state st; xo_seed(&st, seed);
    const double two_pi = 6.283185307179586476925286766559;
    for (long i = 0; i < n; i += 2) {
        double u1 = xo_unit(&st), u2 = xo_unit(&st);
        if (u1 < 1e-300) u1 = 1e-300;
        const double r = sqrt(-2.0 * log(u1));
        out[i] = (float)((double)sigma * r * cos(two_pi * u2));
        if (i + 1 < n) out[i + 1] = (float)((double)sigma * r * sin(two_pi * u2));
    }
}
