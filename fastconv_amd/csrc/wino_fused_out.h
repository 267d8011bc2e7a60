// Output half of the fused Winograd kernels: the 64 per-frequency 32x32 accumulators of a
// workgroup (8 wavefronts x 8 frequencies, MFMA 32x32x2 register layout) are exchanged
// through LDS and turned into 6x6 outputs (+bias, ReLU), written NCHW.
#pragma once

#include "fc_internal.h"
#include "wino_math.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kFW = 8;                      // frequencies per wavefront
constexpr int kFusedThreads = 64 * (64 / kFW);
constexpr size_t kFusedLdsBytes = 64 * 16 * 32 * sizeof(float);   // exchange buffer [64 f][16 k][32 t], 128 KiB

struct FusedOut {
    const float *bias;
    float *y;
    int N, K, OH, OW, relu;
    int tH, tW;
    long T;
    fc_fastdiv divTile, divTW;    // tiles per image, tiles per band
};

// Output channels kb*32 .. kb*32+31, tiles tb*32 .. tb*32+31.  Ml must be free for writing on
// entry (callers put a barrier after their last LDS use).  Accumulator register i of lane l is
// channel 8*(i/4) + 4*(l/32) + i%4, tile l%32: registers 0..7 are channels 0..15, 8..15 are
// 16..31, so the transform runs in two halves of 16 channels.
__device__ __forceinline__ void fused_output_transform(const FusedOut &p, const floatx16 (&acc)[kFW], float *Ml, int kb,
                                                       int tb) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane >> 5, lcol = lane & 31;
    const int tileN = p.tH * p.tW;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        if (half) __syncthreads();
#pragma unroll
        for (int f = 0; f < kFW; f++)
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int krow = 8 * (i / 4) + 4 * lrow + (i % 4);
                Ml[((wave * kFW + f) * 16 + krow) * 32 + lcol] = acc[f][half * 8 + i];
            }
        __syncthreads();
        // one (output channel, tile) pair per thread: 16 x 32 pairs per half
        const int krow = tid >> 5, tl = tid & 31;
        const int k = kb * 32 + half * 16 + krow;
        const uint32_t t = (uint32_t)tb * 32 + tl;
        if (k < p.K && t < (uint32_t)p.T) {
            float m[8][8];
#pragma unroll
            for (int f = 0; f < 64; f++) m[f >> 3][f & 7] = Ml[(f * 16 + krow) * 32 + tl];
            float tmp[6][8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const float col[8] = {m[0][jj], m[1][jj], m[2][jj], m[3][jj], m[4][jj], m[5][jj], m[6][jj], m[7][jj]};
                float sres[6];
                at6(col, sres);
#pragma unroll
                for (int i = 0; i < 6; i++) tmp[i][jj] = sres[i];
            }
            const uint32_t n = fc_div(t, p.divTile), r = t - n * tileN;
            const uint32_t th = fc_div(r, p.divTW), tw = r - th * p.tW;
            const int rows = min(6, p.OH - (int)th * 6), cols = min(6, p.OW - (int)tw * 6);
            const float bias = p.bias ? p.bias[k] : 0.f;
            // ReLU as a maximum with 0, no ReLU as a maximum with -inf: one v_maximum3_f32 either way, which keeps a NaN
            const float floorv = p.relu ? 0.f : -__builtin_inff();
            float *dst = p.y + (((size_t)n * p.K + k) * p.OH + (size_t)th * 6) * p.OW + tw * 6;
            const bool pairs = cols == 6 && (p.OW & 1) == 0;    // 8-byte aligned row segments
#pragma unroll
            for (int i = 0; i < 6; i++) {
                // the bias goes in with element 1 (at6 adds it, as m1 + m2 or m1 - m2, to each output once):
                // the same order of additions as in the staged output transform, whose results this kernel equals bit for bit
                const float rowv[8] = {tmp[i][0], tmp[i][1] + bias, tmp[i][2], tmp[i][3], tmp[i][4], tmp[i][5], tmp[i][6], tmp[i][7]};
                float sres[6];
                at6(rowv, sres);
                if (i < rows) {
#pragma unroll
                    for (int jj = 0; jj < 6; jj++) sres[jj] = __builtin_elementwise_maximum(sres[jj], floorv);
                    float *drow = dst + (size_t)i * p.OW;
                    if (pairs) {
#pragma unroll
                        for (int jj = 0; jj < 6; jj += 2)
                            *reinterpret_cast<float2 *>(drow + jj) = make_float2(sres[jj], sres[jj + 1]);
                    } else {
#pragma unroll
                        for (int jj = 0; jj < 6; jj++)
                            if (jj < cols) drow[jj] = sres[jj];
                    }
                }
            }
        }
    }
}

static inline FusedOut make_fused_out(const fc_wino_plan *plan, const float *bias_dev, int relu, float *y_dev) {
    FusedOut o;
    o.bias = bias_dev; o.y = y_dev;
    o.N = plan->shape.N; o.K = plan->shape.K; o.OH = plan->OH; o.OW = plan->OW; o.relu = relu;
    o.tH = plan->tiles_h; o.tW = plan->tiles_w; o.T = plan->T;
    o.divTile = fc_make_fastdiv((uint32_t)(o.tH * o.tW));
    o.divTW = fc_make_fastdiv((uint32_t)o.tW);
    return o;
}

}  // namespace
