// Whole 3x3 Winograd F(6,3) convolution in one kernel, for layers with few input channels:
// input transform, the 64 per-frequency products and the output transform all happen inside
// a workgroup, so neither V[64][C][T] nor M[64][K][T] (64/36 of the input and of the output
// size, each written and read back by the staged pipeline) ever exists in HBM.
//
// A workgroup owns 16 consecutive tiles x 64 output channels and walks the input channels in
// chunks of 4.  Three chunks are in flight; in every barrier-delimited region each thread
//   1. takes one 8-float row of an 8x8 input patch, fetched two regions earlier as the 8
//      floats of the image row nearest to it (two 16-byte loads, no branches, nothing consumed
//      at load time so the loads stay in flight); rows touching the image border are shifted
//      and zero-filled through a private LDS slot; applies B along the row and parks the
//      result in LDS                                             (tmp[2][4 c][16 t][8][8]),
//   2. applies B^T down one column of the chunk parked in the previous region and writes it as
//      the B operand of the products                             (Vs[2][64 f][4 c][16 t]),
//   3. runs the MFMAs of the chunk transformed in the previous region: wavefront w owns
//      frequencies 8w..8w+7, each a 64x16 accumulator made of four 16x16x4 MFMA blocks; one
//      chunk is one MFMA reduction step.  A comes from the transformed filter in L2 as one
//      16-byte load per frequency and chunk (the four 16-channel blocks of a lane side by
//      side, fetched two regions ahead), B from Vs.
// fp32 MFMA and fp32 vector arithmetic share the SIMD's ALUs on this chip (a measured fact:
// their times add, they do not overlap), so the transform arithmetic is paid on top of the
// products; what the kernel saves is the HBM traffic of V and M.
//
// Filter layout for this kernel ("blocked"): U4[64 f][C_pad/4 q][K_pad/64 kb][4 c][16 k][4 sb]
// holds channel 4q + c, output channel 64kb + 16sb + k: lane (c = l/16, k = l%16) of the MFMA A
// operand finds its four blocks in one 16-byte word and a wavefront reads 1 KiB in one piece.
#include "wino_fused_out.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx4u __attribute__((ext_vector_type(4), aligned(4)));

constexpr int kCB = 4;                          // input channels per chunk
constexpr int kTB = 16;                         // tiles per workgroup
constexpr int kKB = 64;                         // output channels per workgroup
constexpr int kTmpTile = 68;                    // floats per (channel, tile) block of tmp: 16-byte aligned rows,
                                                // 17 quads so that lanes on consecutive tiles spread over the banks
constexpr int kTmpFloats = kCB * kTB * kTmpTile;        // one buffer
constexpr int kVsFreq = 72;                     // floats per frequency of Vs (64 used): 8 banks on, so that the four
                                                // patch columns a half-wavefront stores land in four different bank octets
constexpr int kVsFloats = 64 * kVsFreq;         // one buffer
constexpr int kMlTile = 36;                     // floats per (frequency, tile) of the exchange buffer: 32 channels, padded
constexpr size_t kOnePassLdsBytes = (size_t)64 * kTB * kMlTile * sizeof(float);      // 144 KiB
static_assert((size_t)(2 * kTmpFloats + 2 * kVsFloats + kFusedThreads * 8) * 4 <= kOnePassLdsBytes, "transform buffers must fit under the exchange buffer");

struct OnePassParams {
    const float *x, *U;
    FusedOut out;
    int C, H, W, pad_t, pad_l;
    int K_pad, C_pad;
    int nKB, nTB;
};

__global__ __launch_bounds__(kFusedThreads, 1) void wino_onepass_kernel(const OnePassParams p) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float *tmp = smem;                          // [2][kCB][kTB][kTmpTile]
    float *Vs = smem + 2 * kTmpFloats;          // [2][64][kVsFreq]
    float *bounce = Vs + 2 * kVsFloats;         // [512][8]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // XCD-aware order (workgroup b runs on XCD b % 8): every XCD owns a contiguous range of tile
    // blocks, so the patch rows and columns that neighbouring tiles share -- and the same patches
    // read again by the other output-channel blocks -- are found in that XCD's L2
    const int b = blockIdx.x, xcd = b & 7, jb = b >> 3;
    const int tbl = jb / p.nKB, kb = jb - tbl * p.nKB;
    const int perXcd = (p.nTB + 7) >> 3;
    const int tb = xcd * perXcd + tbl;
    if (tb >= p.nTB) return;

    // ---- step 1: thread = row i1 of the patch of tile tl1, channel c1 of the chunk
    const int tl1 = tid & 15, i1 = (tid >> 4) & 7, c1 = tid >> 7;
    // The row is always fetched as the 8 floats xwin[0..7] that lie inside the image (a window
    // clamped to the row); element j of the patch row is xwin[j + shift] where colMask has bit j.
    const float *xwin = p.x;
    uint32_t colMask = 0;     // bit j: column j of the patch row is inside the image
    int shift = 0;
    {
        const uint32_t t = (uint32_t)tb * kTB + tl1;
        if (t < (uint32_t)p.out.T) {
            const uint32_t n = fc_div(t, p.out.divTile), r = t - n * (p.out.tH * p.out.tW);
            const uint32_t th = fc_div(r, p.out.divTW), tw = r - th * p.out.tW;
            const int gy = (int)th * 6 - p.pad_t + i1, gx0 = (int)tw * 6 - p.pad_l;
            if (gy >= 0 && gy < p.H) {
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (gx0 + j >= 0 && gx0 + j < p.W) colMask |= 1u << j;
                const int gw = min(max(gx0, 0), p.W - 8);       // the host checks W >= 8
                shift = gx0 - gw;
                xwin = p.x + (((size_t)n * p.C + c1) * p.H + gy) * p.W + gw;
            }
        }
    }
    const size_t chunkX = (size_t)kCB * p.H * p.W;
    const int tmpW = (c1 * kTB + tl1) * kTmpTile + i1 * 8;

    // ---- step 2: thread = column j2 of tile tl2, channel c2 (a wavefront: 16 tiles x 4 columns).  Lanes
    // 0..31 hold tiles 0..7 x 4 columns, lanes 32..63 tiles 8..15: with 17 quads per tile in tmp and
    // kVsFreq floats per frequency in Vs, the 32 lanes LDS serves together hit 32 different banks in both.
    const int tl2 = (lane & 7) | ((lane >> 5) << 3), j2 = ((lane >> 3) & 3) + 4 * (wave & 1), c2 = wave >> 1;
    const int tmpR = (c2 * kTB + tl2) * kTmpTile + j2;
    const int vsW = j2 * kVsFreq + c2 * kTB + tl2;            // + 8*kVsFreq per output row

    // ---- step 3
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    const int nq = p.C_pad / kCB;                             // even
    const size_t chunkU = (size_t)p.nKB * 256;                // floats per (frequency, chunk)
    const size_t planeU = (size_t)nq * chunkU;                // floats per frequency
    // wave-uniform base (scalar registers) + one 32-bit lane offset: the filter loads need no address arithmetic
    const float *ub = p.U + (size_t)(wv * kFW) * planeU + (size_t)kb * 256;
    const uint32_t ubLane = (uint32_t)lane * 16u;
    const int vsR = wv * kFW * kVsFreq + lane;                // + kVsFreq per frequency

    floatx4 acc[kFW][4];
#pragma unroll
    for (int f = 0; f < kFW; f++)
#pragma unroll
        for (int sb = 0; sb < 4; sb++) acc[f][sb] = floatx4{0.f, 0.f, 0.f, 0.f};
    floatx4 ua[2][kFW];
    float xr[2][8];

    // Window of chunk q into dst: no branches and nothing consumed here, so the loads stay in
    // flight across regions.  A channel past the last reads (and later discards) the start of x.
    auto loadX = [&](int q, float (&dst)[8]) {
        const float *src = (q * kCB + c1 < p.C) ? xwin + (size_t)q * chunkX : p.x;
        const floatx4u lo = *reinterpret_cast<const floatx4u *>(src);
        const floatx4u hi = *reinterpret_cast<const floatx4u *>(src + 4);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            dst[j] = lo[j];
            dst[4 + j] = hi[j];
        }
    };
    auto loadU = [&](int q, floatx4 (&dst)[kFW]) {
        const float *src = ub + (size_t)q * chunkU;
#pragma unroll
        for (int f = 0; f < kFW; f++)
            dst[f] = *reinterpret_cast<const floatx4 *>(reinterpret_cast<const char *>(src + f * planeU) + ubLane);
    };
    // window (chunk q) -> patch row -> B along the row -> tmp[buf].  Rows that touch the image
    // border are shifted and zero-filled through a private 8-float slot of LDS.
    auto rowTransform = [&](int buf, const float (&win)[8], int q) {
        float d[8], o[8];
#pragma unroll
        for (int j = 0; j < 8; j++) d[j] = win[j];
        const uint32_t m = (q * kCB + c1 < p.C) ? colMask : 0u;
        if (m != 0xffu) {
            float *slot = bounce + tid * 8;
            reinterpret_cast<floatx4 *>(slot)[0] = floatx4{win[0], win[1], win[2], win[3]};
            reinterpret_cast<floatx4 *>(slot)[1] = floatx4{win[4], win[5], win[6], win[7]};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const float v = slot[min(max(j + shift, 0), 7)];
                d[j] = ((m >> j) & 1u) ? v : 0.f;
            }
        }
        bt8(d, o);
        floatx4 *dst = reinterpret_cast<floatx4 *>(tmp + buf * kTmpFloats + tmpW);
        dst[0] = floatx4{o[0], o[1], o[2], o[3]};
        dst[1] = floatx4{o[4], o[5], o[6], o[7]};
    };
    auto colTransform = [&](int buf) {          // tmp[buf] -> Vs[buf]
        const float *src = tmp + buf * kTmpFloats + tmpR;
        float d[8], o[8];
#pragma unroll
        for (int i = 0; i < 8; i++) d[i] = src[i * 8];
        bt8(d, o);
        float *dst = Vs + buf * kVsFloats + vsW;
#pragma unroll
        for (int i = 0; i < 8; i++) dst[i * (8 * kVsFreq)] = o[i];
    };
    float bv[kFW];
    auto loadB = [&](int buf) {
        const float *src = Vs + buf * kVsFloats + vsR;
#pragma unroll
        for (int f = 0; f < kFW; f++) bv[f] = src[f * kVsFreq];
    };
    auto products = [&](const floatx4 (&a)[kFW]) {
#pragma unroll
        for (int f = 0; f < kFW; f++)
#pragma unroll
            for (int sb = 0; sb < 4; sb++)
                acc[f][sb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[f][sb], bv[f], acc[f][sb], 0, 0, 0);
    };

    // prologue: Vs[0] = chunk 0, tmp[1] = rows of chunk 1, xr = rows of chunks 2 and 3, ua = filter chunks 0 and 1
    loadU(0, ua[0]);
    loadU(1, ua[1]);
    loadX(0, xr[0]);
    loadX(1, xr[1]);
    rowTransform(0, xr[0], 0);
    loadX(2, xr[0]);
    __syncthreads();
    colTransform(0);
    rowTransform(1, xr[1], 1);
    loadX(3, xr[1]);
    __syncthreads();

    // region q: rows of chunk q+2 -> tmp[q&1]; columns of chunk q+1: tmp[(q+1)&1] -> Vs[(q+1)&1];
    // products of chunk q out of Vs[q&1]; loads for two regions ahead.  Chunks past the end are
    // zeros and the filter load repeats the last chunk: nothing reads either.
    for (int q = 0; q < nq; q += 2) {
        loadB(0);
        rowTransform(0, xr[0], q + 2);
        colTransform(1);
        products(ua[0]);
        loadU(min(q + 2, nq - 1), ua[0]);
        loadX(q + 4, xr[0]);
        __syncthreads();
        loadB(1);
        rowTransform(1, xr[1], q + 3);
        colTransform(0);
        products(ua[1]);
        loadU(min(q + 3, nq - 1), ua[1]);
        loadX(q + 5, xr[1]);
        __syncthreads();
    }

    // ---- output transform, two halves of 32 output channels through the exchange buffer
    // Ml[64 f][16 t][kMlTile] (32 channels used per tile).  Accumulator block sb, register i of
    // lane l is channel 16*sb + 4*(l/16) + i, tile l%16: the four registers are one 16-byte store.
    float *Ml = smem;
    const int tileN = p.out.tH * p.out.tW;
#pragma unroll
    for (int half = 0; half < 2; half++) {
        if (half) __syncthreads();
#pragma unroll
        for (int f = 0; f < kFW; f++)
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++)
                *reinterpret_cast<floatx4 *>(Ml + ((wave * kFW + f) * 16 + (lane & 15)) * kMlTile + s2 * 16 + 4 * (lane >> 4)) =
                    acc[f][half * 2 + s2];
        __syncthreads();
        // 32 channels x 16 tiles per half; lanes 0..31 of a wavefront hold tiles 0..7 x 4 channels (bank-conflict
        // free reads of the exchange buffer, whose tiles are 36 floats apart)
        const int krow = 4 * wave + ((lane >> 3) & 3), tl = (lane & 7) | ((lane >> 5) << 3);
        const int k = kb * kKB + half * 32 + krow;
        const uint32_t t = (uint32_t)tb * kTB + tl;
        if (k < p.out.K && t < (uint32_t)p.out.T) {
            float m[8][8];
#pragma unroll
            for (int f = 0; f < 64; f++) m[f >> 3][f & 7] = Ml[(f * 16 + tl) * kMlTile + krow];
            float cols[6][8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const float col[8] = {m[0][jj], m[1][jj], m[2][jj], m[3][jj], m[4][jj], m[5][jj], m[6][jj], m[7][jj]};
                float sres[6];
                at6(col, sres);
#pragma unroll
                for (int i = 0; i < 6; i++) cols[i][jj] = sres[i];
            }
            const uint32_t n = fc_div(t, p.out.divTile), r = t - n * tileN;
            const uint32_t th = fc_div(r, p.out.divTW), tw = r - th * p.out.tW;
            const int rows = min(6, p.out.OH - (int)th * 6), ncols = min(6, p.out.OW - (int)tw * 6);
            const float bias = p.out.bias ? p.out.bias[k] : 0.f;
            float *dst = p.out.y + (((size_t)n * p.out.K + k) * p.out.OH + (size_t)th * 6) * p.out.OW + tw * 6;
            const bool pairs = ncols == 6 && (p.out.OW & 1) == 0;    // 8-byte aligned row segments
#pragma unroll
            for (int i = 0; i < 6; i++) {
                float sres[6];
                at6(cols[i], sres);
                if (i < rows) {
#pragma unroll
                    for (int jj = 0; jj < 6; jj++) {
                        sres[jj] += bias;
                        if (p.out.relu) sres[jj] = __builtin_elementwise_maximum(sres[jj], 0.f);      // keeps a NaN, as the other epilogues do
                    }
                    float *drow = dst + (size_t)i * p.out.OW;
                    if (pairs) {
#pragma unroll
                        for (int jj = 0; jj < 6; jj += 2)
                            *reinterpret_cast<float2 *>(drow + jj) = make_float2(sres[jj], sres[jj + 1]);
                    } else {
#pragma unroll
                        for (int jj = 0; jj < 6; jj++)
                            if (jj < ncols) drow[jj] = sres[jj];
                    }
                }
            }
        }
    }
}

// Filter transform into the blocked layout; one thread per (output channel, input channel).
__global__ __launch_bounds__(256) void wino_filter_transform_blocked_kernel(const float *__restrict__ w, float *__restrict__ U,
                                                                            int K, int C, int K_pad, int C_pad) {
    const int k = blockIdx.x * 64 + (threadIdx.x & 63);
    const int c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (k >= K_pad || c >= C_pad) return;
    float g[3][3];
#pragma unroll
    for (int i = 0; i < 9; i++) g[i / 3][i % 3] = (k < K && c < C) ? w[((size_t)k * C + c) * 9 + i] : 0.f;
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
    const int nKB = K_pad / 64;
    const int q = c >> 2, cc = c & 3, kb = k >> 6, sb = (k >> 4) & 3, k16 = k & 15;
    float *dst = U + ((((size_t)q * nKB + kb) * 4 + cc) * 16 + k16) * 4 + sb;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float o[8];
        g8(t[i], o);
#pragma unroll
        for (int j = 0; j < 8; j++) dst[(size_t)(i * 8 + j) * plane] = o[j];
    }
}

int onepass_plan_check(fc_context *ctx, const fc_wino_plan *plan, const void *a, const void *b) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !a || !b) return fc_set_error(ctx, FC_ERR_INVALID, "null plan or buffer", hipSuccess);
    fc_wino_plan chk;
    const int rc = fc_wino_make_onepass_plan(&plan->shape, &chk);
    if (rc) return fc_set_error(ctx, rc, "plan does not describe a layer the single-kernel path supports", hipSuccess);
    if (plan->gemm_config != FC_WINO_ONEPASS || !fc_same_wino_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "not a plan made by fc_wino_make_onepass_plan", hipSuccess);
    return FC_OK;
}

}  // namespace

extern "C" int fc_wino_make_onepass_plan(const fc_conv_shape *s, fc_wino_plan *plan) {
    if (!plan || !fc_shape_ok(s)) return FC_ERR_INVALID;
    if (s->kh != 3 || s->kw != 3 || s->sh != 1 || s->sw != 1) return FC_ERR_INVALID;
    plan->shape = *s;
    plan->OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1);
    plan->OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    plan->tiles_h = (plan->OH + 5) / 6;
    plan->tiles_w = (plan->OW + 5) / 6;
    plan->T = (long)s->N * plan->tiles_h * plan->tiles_w;
    plan->K_pad = (int)fc_round_up(s->K, kKB);
    plan->C_pad = (int)fc_round_up(s->C, 2 * kCB);
    plan->T_pad = fc_round_up(plan->T, kTB);
    plan->gemm_config = FC_WINO_ONEPASS;
    plan->U_bytes = sizeof(float) * 64 * (size_t)plan->C_pad * plan->K_pad;
    plan->V_bytes = 0;
    plan->M_bytes = 0;
    if (plan->T_pad >= (1l << 31) || (long)s->N * s->C * s->H * s->W >= (1l << 40)) return FC_ERR_UNSUPPORTED;
    if (s->W < 8) return FC_ERR_UNSUPPORTED;      // a patch row is fetched as 8 floats of one image row
    return FC_OK;
}

extern "C" int fc_wino_onepass_filter_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev,
                                                float *U_dev) {
    const int rc = onepass_plan_check(ctx, plan, w_dev, U_dev);
    if (rc) return rc;
    if (fc_wino_smallc_applies(&plan->shape)) return fc_wino_smallc_filter_transform(ctx, plan, w_dev, U_dev);
    const dim3 grid((plan->K_pad + 63) / 64, (plan->C_pad + 3) / 4);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_onepass_filter_transform: too many channels", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_KERNEL_TRAN);
    wino_filter_transform_blocked_kernel<<<grid, dim3(256), 0, ctx->stream>>>(w_dev, U_dev, plan->shape.K, plan->shape.C,
                                                                            plan->K_pad, plan->C_pad);
    FC_LAUNCH_CHECK(ctx, "wino_filter_transform_blocked_kernel");
    return FC_OK;
}

extern "C" int fc_wino_conv_onepass(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, const float *U_dev,
                                    const float *bias_dev, int relu, float *y_dev) {
    int rc = onepass_plan_check(ctx, plan, x_dev, U_dev);
    if (rc) return rc;
    if (!y_dev) return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_conv_onepass: null output", hipSuccess);
    if (((uintptr_t)y_dev & 7) != 0 || ((uintptr_t)U_dev & 15) != 0 || ((uintptr_t)x_dev & 3) != 0)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_conv_onepass: y must be 8-byte and U 16-byte aligned", hipSuccess);
    if (fc_wino_smallc_applies(&plan->shape))
        return fc_wino_smallc_conv(ctx, plan, x_dev, const_cast<float *>(U_dev), nullptr, bias_dev, relu, y_dev);
    if (!ctx->onepass_lds_granted) {
        if (ctx->capturing)
            return fc_set_error(ctx, FC_ERR_STATE, "fc_wino_conv_onepass: run this kernel once before recording a graph with it", hipSuccess);
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_onepass_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)kOnePassLdsBytes));
        ctx->onepass_lds_granted = true;
    }
    const fc_conv_shape &s = plan->shape;
    OnePassParams p;
    p.x = x_dev; p.U = U_dev;
    p.out = make_fused_out(plan, bias_dev, relu, y_dev);
    p.C = s.C; p.H = s.H; p.W = s.W; p.pad_t = s.pt; p.pad_l = s.pl;
    p.K_pad = plan->K_pad; p.C_pad = plan->C_pad;
    p.nKB = plan->K_pad / kKB;
    p.nTB = (int)((plan->T + kTB - 1) / kTB);
    const long blocks = (long)((p.nTB + 7) / 8) * 8 * p.nKB;
    if (blocks >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_conv_onepass: grid too large", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_ONEPASS);
    wino_onepass_kernel<<<dim3((unsigned)blocks), dim3(kFusedThreads), kOnePassLdsBytes, ctx->stream>>>(p);
    FC_LAUNCH_CHECK(ctx, "wino_onepass_kernel");
    return FC_OK;
}

extern "C" int fc_wino_prefer_onepass(const fc_conv_shape *s) {
    if (!fc_shape_ok(s) || s->kh != 3 || s->kw != 3 || s->sh != 1 || s->sw != 1 || s->W < 8) return 0;
    // at most four channels: a kernel of its own on the vector ALUs, the fastest Winograd path at every batch
    if (fc_wino_smallc_applies(s)) return 1;
    if (s->C < 16 || s->C > 64) return 0;
    // one 16-tile x 64-channel block per workgroup, one workgroup per CU at a time: the layer must
    // bring a few blocks per CU (batch 1 layers do not).  Measured crossover against the staged
    // pipeline: about 200 blocks when one block covers all output channels, 500 otherwise.
    const long OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1), OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    const long blocks = ((long)s->N * ((OH + 5) / 6) * ((OW + 5) / 6) + kTB - 1) / kTB * ((s->K + kKB - 1) / kKB);
    return blocks >= (s->K <= kKB ? 192 : 512) ? 1 : 0;
}

extern "C" int fc_wino_forward_onepass(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, const float *w_dev,
                                       const float *bias_dev, int relu, int filter_ready, float *U_dev, float *y_dev) {
    if (!filter_ready) {
        int rc = onepass_plan_check(ctx, plan, w_dev, U_dev);
        if (rc) return rc;
        if (fc_wino_smallc_applies(&plan->shape) && fc_wino_smallc_transforms_inside(ctx, plan)) {
            // few tiles: one launch, the filter is transformed by the wavefronts that use it (and U filled all the same)
            rc = onepass_plan_check(ctx, plan, x_dev, U_dev);
            if (rc) return rc;
            if (!y_dev) return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_forward_onepass: null output", hipSuccess);
            if (((uintptr_t)y_dev & 7) != 0 || ((uintptr_t)U_dev & 15) != 0 || ((uintptr_t)x_dev & 3) != 0 || ((uintptr_t)w_dev & 3) != 0)
                return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_forward_onepass: y must be 8-byte and U 16-byte aligned", hipSuccess);
            return fc_wino_smallc_conv(ctx, plan, x_dev, U_dev, w_dev, bias_dev, relu, y_dev);
        }
        rc = fc_wino_onepass_filter_transform(ctx, plan, w_dev, U_dev);
        if (rc) return rc;
    }
    return fc_wino_conv_onepass(ctx, plan, x_dev, U_dev, bias_dev, relu, y_dev);
}
