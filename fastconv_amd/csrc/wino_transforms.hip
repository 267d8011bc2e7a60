// Winograd F(6x6,3x3) transform kernels for gfx950: filter (G g G^T), input
// (B^T d B) and output (A^T m A).  All three are HBM-bound; the layouts are
//   U[64][C_pad][K_pad], V[64][C_pad][T_pad], M[64][K_pad][T_pad]
// with the last index fastest, so that a wavefront whose lanes walk consecutive
// output channels (U) or consecutive tiles (V, M) touches 256 contiguous bytes
// per frequency plane.
#include "fc_internal.h"

namespace {

// ---- 1-D transforms (the matrices of winoF63ZC/winoF63ZC.cpp:28-78,
// :137-166 and :181-228, factored by common sub-expressions) ---------------

__device__ __forceinline__ void bt8(const float d[8], float o[8]) {
    o[0] = (d[0] - d[6]) + 5.25f * (d[4] - d[2]);
    o[7] = (d[7] - d[1]) + 5.25f * (d[3] - d[5]);
    const float t1 = (d[2] + d[6]) - 4.25f * d[4];
    const float t2 = (d[1] + d[5]) - 4.25f * d[3];
    o[1] = t1 + t2;
    o[2] = t1 - t2;
    const float p1 = (d[6] + 0.25f * d[2]) - 1.25f * d[4];
    const float p2 = (0.5f * d[1] - 2.5f * d[3]) + 2.0f * d[5];
    o[3] = p1 + p2;
    o[4] = p1 - p2;
    const float q1 = (d[6] + 4.0f * d[2]) - 5.0f * d[4];
    const float q2 = (2.0f * d[1] - 2.5f * d[3]) + 0.5f * d[5];
    o[5] = q1 + q2;
    o[6] = q1 - q2;
}

__device__ __forceinline__ void at6(const float m[8], float s[6]) {
    const float a = m[1] + m[2], b = m[1] - m[2];
    const float c = m[3] + m[4], d = m[3] - m[4];
    const float e = m[5] + m[6], f = m[5] - m[6];
    s[0] = (m[0] + a) + (c + 32.0f * e);
    s[1] = (b + 2.0f * d) + 16.0f * f;
    s[2] = (a + 4.0f * c) + 8.0f * e;
    s[3] = (b + 8.0f * d) + 4.0f * f;
    s[4] = (a + 16.0f * c) + 2.0f * e;
    s[5] = ((b + 32.0f * d) + f) + m[7];
}

__device__ __forceinline__ void g8(const float g[3], float w[8]) {
    const float c29 = (float)(-2.0 / 9), c90 = (float)(1.0 / 90), c180 = (float)(1.0 / 180);
    const float s02 = g[0] + g[2];
    w[0] = g[0];
    w[1] = (s02 + g[1]) * c29;
    w[2] = (s02 - g[1]) * c29;
    const float e = g[0] + 4.0f * g[2], two = 2.0f * g[1];
    w[3] = (e + two) * c90;
    w[4] = (e - two) * c90;
    const float h = g[2] + 4.0f * g[0];
    w[5] = (h + two) * c180;
    w[6] = (h - two) * c180;
    w[7] = g[2];
}

// ---------------------------------------------------------------- filter

// One thread per (output channel, input channel); lanes walk output channels so
// the 64 plane stores of a wavefront are contiguous.
__global__ __launch_bounds__(256) void wino_filter_transform_kernel(const float *__restrict__ w,
                                                                    float *__restrict__ U, int K, int C,
                                                                    int K_pad, int C_pad) {
    const int k = blockIdx.x * 64 + (threadIdx.x & 63);
    const int c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (k >= K_pad || c >= C_pad) return;
    float g[3][3];
    if (k < K && c < C) {
        const float *src = w + ((size_t)k * C + c) * 9;
#pragma unroll
        for (int i = 0; i < 9; i++) g[i / 3][i % 3] = src[i];
    } else {
#pragma unroll
        for (int i = 0; i < 9; i++) g[i / 3][i % 3] = 0.f;
    }
    // columns first: t[:, j] = G g[:, j]
    float t[8][3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        const float col[3] = {g[0][j], g[1][j], g[2][j]};
        float o[8];
        g8(col, o);
#pragma unroll
        for (int i = 0; i < 8; i++) t[i][j] = o[i];
    }
    const size_t plane = (size_t)C_pad * K_pad;
    float *dst = U + (size_t)c * K_pad + k;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float o[8];
        g8(t[i], o);
#pragma unroll
        for (int j = 0; j < 8; j++) dst[(size_t)(i * 8 + j) * plane] = o[j];
    }
}

// ----------------------------------------------------------------- input

struct InTParams {
    const float *x;
    float *V;
    int N, C, H, W, pad_t, pad_l;
    int tH, tW, tileN;
    long T;
    int C_pad;
    long T_pad;
    int P, R;        // images and tile rows ("bands") per block; a block always spans all tW columns
    int nPG, nBG;    // groups of images, groups of bands
    int LW;          // 6*tW + 2 columns of the band as the tiles see it (incl. padding columns)
    fc_fastdiv divLW, divR, divTW;
};

// Block = one input channel x (P images x R bands x tW tiles), TPB tiles at most.
// Pass 1 applies B^T down the 8 rows of each band: a thread owns one column of
// one band, so the 8 global loads of a wavefront are row-contiguous.  Pass 2
// applies B along the rows from LDS: a thread owns one tile (and 8*TPB/256 of
// its 8 rows) and stores to the frequency planes with lanes on consecutive
// tiles.  The extra last block in x zero-fills the tile padding [T, T_pad).
template <int TPB>
__global__ __launch_bounds__(256) void wino_input_transform_kernel(const InTParams p) {
    extern __shared__ float lds[];   // [P*R][8][LW]
    const int tid = threadIdx.x;
    const int c = blockIdx.y;
    const size_t plane = (size_t)p.C_pad * p.T_pad;
    const int nChunks = p.nPG * p.nBG;

    if ((int)blockIdx.x == nChunks) {
        const long padT = p.T_pad - p.T;
        for (long e = tid; e < padT * 64; e += 256) {
            const long f = e / padT, t = p.T + (e - f * padT);
            p.V[f * plane + (size_t)c * p.T_pad + t] = 0.f;
        }
        return;
    }
    const int pg = blockIdx.x / p.nBG, bg = blockIdx.x - pg * p.nBG;
    const int n0 = pg * p.P, th0 = bg * p.R;
    const int PR = p.P * p.R;

    if (c < p.C) {
        const int items = PR * p.LW;
        for (int e = tid; e < items; e += 256) {
            const int pr = fc_div(e, p.divLW), lx = e - pr * p.LW;
            const int pp = fc_div(pr, p.divR), r = pr - pp * p.R;
            const int n = n0 + pp, th = th0 + r;
            if (n >= p.N || th >= p.tH) continue;
            const int gx = lx - p.pad_l, gy0 = th * 6 - p.pad_t;
            float d[8], o[8];
            const bool colOK = gx >= 0 && gx < p.W;
            const float *src = p.x + (((size_t)n * p.C + c) * p.H) * p.W + gx;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const int gy = gy0 + i;
                d[i] = (colOK && gy >= 0 && gy < p.H) ? src[(long)gy * p.W] : 0.f;
            }
            bt8(d, o);
            float *dstl = lds + (size_t)pr * 8 * p.LW + lx;
#pragma unroll
            for (int i = 0; i < 8; i++) dstl[i * p.LW] = o[i];
        }
    }
    __syncthreads();

    constexpr int IPT = 8 * TPB / 256;     // rows of the 8x8 tile per thread
    const int tl = tid % TPB, ig = tid / TPB;
    const int pr = fc_div(tl, p.divTW), q = tl - pr * p.tW;
    if (pr >= PR) return;
    const int pp = fc_div(pr, p.divR), r = pr - pp * p.R;
    const int n = n0 + pp, th = th0 + r;
    if (n >= p.N || th >= p.tH) return;
    const long t = (long)n * p.tileN + (long)th * p.tW + q;
    float *dst = p.V + (size_t)c * p.T_pad + t;
    if (c < p.C) {
#pragma unroll
        for (int ii = 0; ii < IPT; ii++) {
            const int i = ig * IPT + ii;
            const float *row = lds + ((size_t)pr * 8 + i) * p.LW + q * 6;
            float d[8], o[8];
#pragma unroll
            for (int j = 0; j < 8; j++) d[j] = row[j];
            bt8(d, o);
#pragma unroll
            for (int j = 0; j < 8; j++) dst[(size_t)(i * 8 + j) * plane] = o[j];
        }
    } else {
#pragma unroll
        for (int ii = 0; ii < IPT; ii++) {
            const int i = ig * IPT + ii;
#pragma unroll
            for (int j = 0; j < 8; j++) dst[(size_t)(i * 8 + j) * plane] = 0.f;
        }
    }
}

// ---------------------------------------------------------------- output

struct OutTParams {
    const float *M;
    const float *bias;
    float *y;
    int N, K, OH, OW, relu;
    int tH, tW, tileN;
    int K_pad;
    long T_pad;
    int P, R, nPG, nBG;
    fc_fastdiv divR, divTW;
};

// Block = one output channel x (P images x R bands x tW tiles); one thread per
// tile.  The 64 plane loads of a wavefront are each 256 contiguous bytes.  The
// 6x6 results are laid into LDS as the exact image rows they cover and copied
// out as one contiguous run per image.
template <int TPB>
__global__ __launch_bounds__(TPB) void wino_output_transform_kernel(const OutTParams p) {
    extern __shared__ float lds[];   // [P][rows*OW]
    const int tid = threadIdx.x;
    const int k = blockIdx.y;
    const int pg = blockIdx.x / p.nBG, bg = blockIdx.x - pg * p.nBG;
    const int n0 = pg * p.P, th0 = bg * p.R;
    const int row0 = th0 * 6;
    const int rows = min(p.R * 6, p.OH - row0);      // output rows this block covers
    const int L = rows * p.OW;                       // floats per image in this block

    const int pr = fc_div(tid, p.divTW), q = tid - pr * p.tW;
    const int pp = fc_div(pr, p.divR), r = pr - pp * p.R;
    const int n = n0 + pp, th = th0 + r;
    if (pr < p.P * p.R && n < p.N && th < p.tH) {
        const size_t plane = (size_t)p.K_pad * p.T_pad;
        const long t = (long)n * p.tileN + (long)th * p.tW + q;
        const float *src = p.M + (size_t)k * p.T_pad + t;
        float m[8][8];
#pragma unroll
        for (int f = 0; f < 64; f++) m[f >> 3][f & 7] = src[(size_t)f * plane];
        float tmp[6][8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float col[8] = {m[0][j], m[1][j], m[2][j], m[3][j], m[4][j], m[5][j], m[6][j], m[7][j]};
            float s[6];
            at6(col, s);
#pragma unroll
            for (int i = 0; i < 6; i++) tmp[i][j] = s[i];
        }
        const float b = p.bias ? p.bias[k] : 0.f;
        float *img = lds + (size_t)pp * L;
        const int colBase = q * 6;
#pragma unroll
        for (int i = 0; i < 6; i++) {
            float s[6];
            at6(tmp[i], s);
            const int lr = r * 6 + i;
            if (lr < rows) {
#pragma unroll
                for (int j = 0; j < 6; j++) {
                    float v = s[j] + b;
                    if (p.relu) v = fmaxf(v, 0.f);
                    if (colBase + j < p.OW) img[lr * p.OW + colBase + j] = v;
                }
            }
        }
    }
    __syncthreads();
    const int nImg = min(p.P, p.N - n0);
    const size_t imgStride = (size_t)p.K * p.OH * p.OW;
    float *dst0 = p.y + ((size_t)n0 * p.K + k) * p.OH * p.OW + (size_t)row0 * p.OW;
    for (int pi = 0; pi < nImg; pi++) {
        const float *img = lds + (size_t)pi * L;
        float *dst = dst0 + (size_t)pi * imgStride;
        for (int e = tid; e < L; e += TPB) dst[e] = img[e];
    }
}

// Choose images (P) and bands (R) per block for `tpb` tiles per block.
bool chunking(int tpb, int N, int tH, int tW, int *P, int *R) {
    const int tileN = tH * tW;
    if (tW > tpb) return false;
    if (tileN <= tpb) {
        *R = tH;
        *P = tpb / tileN;
        if (*P > N) *P = N;
    } else {
        *P = 1;
        *R = tpb / tW;
    }
    return true;
}

}  // namespace

// ------------------------------------------------------------------ host

extern "C" int fc_wino_make_plan(const fc_conv_shape *s, int gemm_config, fc_wino_plan *plan) {
    if (!plan || !fc_shape_ok(s)) return FC_ERR_INVALID;
    if (s->kh != 3 || s->kw != 3 || s->sh != 1 || s->sw != 1) return FC_ERR_INVALID;
    fc_gemm_config cfg;
    const int rc = fc_wino_gemm_get_config(gemm_config, &cfg);
    if (rc) return rc;
    plan->shape = *s;
    plan->OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1);
    plan->OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    plan->tiles_h = (plan->OH + 5) / 6;
    plan->tiles_w = (plan->OW + 5) / 6;
    plan->T = (long)s->N * plan->tiles_h * plan->tiles_w;
    plan->K_pad = (int)fc_round_up(s->K, cfg.bm);
    plan->C_pad = (int)fc_round_up(s->C, cfg.bk);
    plan->T_pad = fc_round_up(plan->T, cfg.bn);
    plan->gemm_config = gemm_config;
    plan->U_bytes = sizeof(float) * 64 * (size_t)plan->C_pad * plan->K_pad;
    plan->V_bytes = sizeof(float) * 64 * (size_t)plan->C_pad * plan->T_pad;
    plan->M_bytes = sizeof(float) * 64 * (size_t)plan->K_pad * plan->T_pad;
    if (plan->tiles_w > 256) return FC_ERR_UNSUPPORTED;       // output wider than 1536
    if (plan->T_pad >= (1l << 31) || (size_t)plan->C_pad * plan->T_pad >= (1ull << 31) ||
        (size_t)plan->K_pad * plan->T_pad >= (1ull << 31))
        return FC_ERR_UNSUPPORTED;
    return FC_OK;
}

static int plan_check(fc_context *ctx, const fc_wino_plan *plan, const void *a, const void *b) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !a || !b) return fc_set_error(ctx, FC_ERR_INVALID, "null plan or buffer", hipSuccess);
    fc_wino_plan chk;
    const int rc = fc_wino_make_plan(&plan->shape, plan->gemm_config, &chk);
    if (rc) return fc_set_error(ctx, rc, "plan does not describe a supported layer", hipSuccess);
    if (chk.K_pad != plan->K_pad || chk.C_pad != plan->C_pad || chk.T_pad != plan->T_pad || chk.T != plan->T)
        return fc_set_error(ctx, FC_ERR_INVALID, "plan fields were modified after fc_wino_make_plan", hipSuccess);
    return FC_OK;
}

extern "C" int fc_wino_filter_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev,
                                        float *U_dev) {
    const int rc = plan_check(ctx, plan, w_dev, U_dev);
    if (rc) return rc;
    const dim3 grid((plan->K_pad + 63) / 64, (plan->C_pad + 3) / 4);
    fc_stage_scope scope(ctx, FC_STAGE_KERNEL_TRAN);
    wino_filter_transform_kernel<<<grid, dim3(256), 0, ctx->stream>>>(w_dev, U_dev, plan->shape.K, plan->shape.C,
                                                                     plan->K_pad, plan->C_pad);
    FC_LAUNCH_CHECK(ctx, "wino_filter_transform_kernel");
    return FC_OK;
}

extern "C" int fc_wino_input_transform(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                                       float *V_dev) {
    const int rc = plan_check(ctx, plan, x_dev, V_dev);
    if (rc) return rc;
    const fc_conv_shape &s = plan->shape;
    InTParams p;
    p.x = x_dev; p.V = V_dev;
    p.N = s.N; p.C = s.C; p.H = s.H; p.W = s.W; p.pad_t = s.pt; p.pad_l = s.pl;
    p.tH = plan->tiles_h; p.tW = plan->tiles_w; p.tileN = p.tH * p.tW;
    p.T = plan->T; p.C_pad = plan->C_pad; p.T_pad = plan->T_pad;
    p.LW = 6 * p.tW + 2;
    // pick the tiles-per-block variant that wastes the fewest lanes and fits 64 KiB of LDS
    int best = 0, bestP = 0, bestR = 0;
    double bestUtil = -1.0;
    const int cand[3] = {64, 128, 256};
    for (int i = 0; i < 3; i++) {
        int P, R;
        if (!chunking(cand[i], s.N, p.tH, p.tW, &P, &R)) continue;
        const size_t ldsBytes = (size_t)P * R * 8 * p.LW * sizeof(float);
        if (ldsBytes > 64 * 1024) continue;
        const int nBG = (p.tH + R - 1) / R;
        // average fraction of busy lanes over the band groups of one image group
        const double util = (double)p.tH * p.tW * P / ((double)nBG * cand[i]);
        if (util > bestUtil + 0.02) { bestUtil = util; best = cand[i]; bestP = P; bestR = R; }
    }
    if (!best) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: image too wide", hipSuccess);
    p.P = bestP; p.R = bestR;
    p.nPG = (s.N + p.P - 1) / p.P;
    p.nBG = (p.tH + p.R - 1) / p.R;
    p.divLW = fc_make_fastdiv(p.LW);
    p.divR = fc_make_fastdiv(p.R);
    p.divTW = fc_make_fastdiv(p.tW);
    const size_t ldsBytes = (size_t)p.P * p.R * 8 * p.LW * sizeof(float);
    const dim3 grid(p.nPG * p.nBG + 1, plan->C_pad);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: more than 65535 channels", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_INPUT_TRAN);
    if (best == 64) wino_input_transform_kernel<64><<<grid, dim3(256), ldsBytes, ctx->stream>>>(p);
    else if (best == 128) wino_input_transform_kernel<128><<<grid, dim3(256), ldsBytes, ctx->stream>>>(p);
    else wino_input_transform_kernel<256><<<grid, dim3(256), ldsBytes, ctx->stream>>>(p);
    FC_LAUNCH_CHECK(ctx, "wino_input_transform_kernel");
    return FC_OK;
}

extern "C" int fc_wino_output_transform(fc_context *ctx, const fc_wino_plan *plan, const float *M_dev,
                                        const float *bias_dev, int relu, float *y_dev) {
    const int rc = plan_check(ctx, plan, M_dev, y_dev);
    if (rc) return rc;
    const fc_conv_shape &s = plan->shape;
    OutTParams p;
    p.M = M_dev; p.bias = bias_dev; p.y = y_dev;
    p.N = s.N; p.K = s.K; p.OH = plan->OH; p.OW = plan->OW; p.relu = relu;
    p.tH = plan->tiles_h; p.tW = plan->tiles_w; p.tileN = p.tH * p.tW;
    p.K_pad = plan->K_pad; p.T_pad = plan->T_pad;
    int best = 0, bestP = 0, bestR = 0;
    double bestUtil = -1.0;
    const int cand[3] = {64, 128, 256};
    for (int i = 0; i < 3; i++) {
        int P, R;
        if (!chunking(cand[i], s.N, p.tH, p.tW, &P, &R)) continue;
        const int nBG = (p.tH + R - 1) / R;
        const double util = (double)p.tH * p.tW * P / ((double)nBG * cand[i]);
        if (util > bestUtil + 0.02) { bestUtil = util; best = cand[i]; bestP = P; bestR = R; }
    }
    if (!best) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_output_transform: image too wide", hipSuccess);
    p.P = bestP; p.R = bestR;
    p.nPG = (s.N + p.P - 1) / p.P;
    p.nBG = (p.tH + p.R - 1) / p.R;
    p.divR = fc_make_fastdiv(p.R);
    p.divTW = fc_make_fastdiv(p.tW);
    const size_t ldsBytes = (size_t)p.P * min(p.R * 6, p.OH) * p.OW * sizeof(float);
    const dim3 grid(p.nPG * p.nBG, s.K);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_output_transform: more than 65535 channels", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_OUTPUT_TRAN);
    if (best == 64) wino_output_transform_kernel<64><<<grid, dim3(64), ldsBytes, ctx->stream>>>(p);
    else if (best == 128) wino_output_transform_kernel<128><<<grid, dim3(128), ldsBytes, ctx->stream>>>(p);
    else wino_output_transform_kernel<256><<<grid, dim3(256), ldsBytes, ctx->stream>>>(p);
    FC_LAUNCH_CHECK(ctx, "wino_output_transform_kernel");
    return FC_OK;
}

extern "C" int fc_wino_forward(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, const float *w_dev,
                               const float *bias_dev, int relu, int filter_ready, float *U_dev, float *V_dev,
                               float *M_dev, float *y_dev) {
    int rc;
    if (!filter_ready) {
        rc = fc_wino_filter_transform(ctx, plan, w_dev, U_dev);
        if (rc) return rc;
    }
    rc = fc_wino_input_transform(ctx, plan, x_dev, V_dev);
    if (rc) return rc;
    rc = fc_wino_gemm(ctx, plan, U_dev, V_dev, M_dev);
    if (rc) return rc;
    return fc_wino_output_transform(ctx, plan, M_dev, bias_dev, relu, y_dev);
}
