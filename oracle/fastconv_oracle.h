/*
 * CPU oracle for the FastConv convolution hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * algorithms, used as the checker by tests/, by __graft_entry__.smoke() and by
 * the cpu_baseline leg of bench.py.  Nothing in the shipped library or in the
 * C++ host layers links, loads or calls it.
 *
 * Every function names the reference file:line it restates (paths relative to
 * the reference checkout).  The reference has no batch dimension; here a
 * leading N is a plain outer loop over independent images.
 *
 * How each function is pinned (tests/test_oracle.py):
 *   fco_naive_conv_f32 / _f64  against the reference's own naive layers built
 *                              from source (oracle/_ref), closed forms
 *                              (all-ones, delta and shift kernels), linearity
 *   fco_wino_*                 brute-force 8x8 (*) 3x3 valid correlation per
 *                              tile, matrix tables, agreement with the naive
 *                              conv on edge shapes
 *   fco_im2col / fco_sgemm     agreement with the naive conv, hand-counted
 *                              small cases
 *   fco_diff_legacy            hand-computed vectors
 *   fco_rng_*                  published splitmix64 / xoshiro256** outputs
 */
#ifndef FASTCONV_ORACLE_H_
#define FASTCONV_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int N, C, H, W;        /* input  N x C x H x W, fp32 NCHW            */
    int K, kh, kw;         /* filter K x C x kh x kw                     */
    int sh, sw;            /* stride                                     */
    int pt, pb, pl, pr;    /* padding top / bottom / left / right        */
} fco_shape;

/* conv_layer.h:68-69 */
int fco_out_h(const fco_shape *s);
int fco_out_w(const fco_shape *s);

/* bias_mode: 0 none, 1 per output channel [K], 2 per output element
 * [K*OH*OW] (the form convLayer/naiveConv_wudu.h:78 adds). */
int fco_naive_conv_f32(const fco_shape *s, const float *x, const float *w,
                       const float *bias, int bias_mode, float *y);
int fco_naive_conv_f64(const fco_shape *s, const float *x, const float *w,
                       const float *bias, int bias_mode, double *y);

/* Winograd F(6x6,3x3).  Frequencies are numbered f = 8*row + col of the
 * transformed 8x8 tile.  Tiles are numbered t = (n*tileH + th)*tileW + tw. */
int fco_wino_tiles_h(const fco_shape *s);
int fco_wino_tiles_w(const fco_shape *s);
void fco_wino_matrices(float BT[64], float G[24], float AT[48]);
/* U[f][k][c] */
int fco_wino_filter_transform(const float *w, float *U, int K, int C);
/* V[f][c][t] */
int fco_wino_input_transform(const fco_shape *s, const float *x, float *V);
/* M[f][k][t] = sum_c U[f][k][c] * V[f][c][t] */
int fco_wino_gemm(const float *U, const float *V, float *M, int K, int C, long T);
int fco_wino_output_transform(const fco_shape *s, const float *M,
                              const float *bias, float *y);
int fco_wino_conv_f32(const fco_shape *s, const float *x, const float *w,
                      const float *bias, float *y);

/* im2col + GEMM.  col is [C*kh*kw][N*OH*OW]. */
int fco_im2col(const fco_shape *s, const float *x, float *col);
void fco_sgemm(int M, long Ncols, int Kred, const float *A, const float *B, float *Cmat);
int fco_im2col_conv_f32(const fco_shape *s, const float *x, const float *w,
                        const float *bias, float *y);

/* utility/helper.cpp:74-89 */
float fco_diff_legacy(const float *a, const float *b, long len);
/* max_i |y_i - ref_i| / max_i |ref_i| */
double fco_max_rel_err_f32(const float *y, const double *ref, long len);
double fco_max_rel_err_f32f32(const float *y, const float *ref, long len);

/* splitmix64-seeded xoshiro256**; uniform on [lo,hi), normal by Box-Muller in
 * double then rounded to float. */
void fco_rng_raw(uint64_t seed, uint64_t *out, long n);
void fco_rng_uniform(uint64_t seed, float lo, float hi, float *out, long n);
void fco_rng_normal(uint64_t seed, float sigma, float *out, long n);

int fco_num_threads(void);

#ifdef __cplusplus
}
#endif
#endif
