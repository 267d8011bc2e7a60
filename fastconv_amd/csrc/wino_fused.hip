// Winograd GEMM and output transform in one kernel, for layers whose transformed
// filter stays in L2 (few channels): the 64 per-frequency products of a
// (32 output channels x 32 tiles) block are accumulated in registers, exchanged
// through LDS and turned into 6x6 outputs, so M[64][K][T] -- 64/36 of the output
// size, written and read back by the staged pipeline -- never exists in HBM.
//
// A workgroup is 8 wavefronts (two per SIMD, so each hides the other's latencies);
// wavefront w owns frequencies 8w..8w+7, i.e. 8 independent 32x32 MFMA
// accumulators (128 accumulation registers).  Nothing is
// shared between wavefronts during the reduction, so operands go straight from
// global memory (L2) to registers: for reduction step (c, c+1) lane l of each
// frequency loads U[f][c + l/32][k0 + l%32] and V[f][c + l/32][t0 + l%32], two
// full 128-byte lines per load instruction.  Loads run three steps ahead.
#include "wino_fused_out.h"

namespace {

struct FusedParams {
    const float *U, *V;
    FusedOut out;
    int K_pad, C_pad;
    long T_pad;
    int nKB, nTB;
};

// uniform base + 32-bit lane offset in bytes: the scalar-base form of global_load
__device__ __forceinline__ float ldg(const float *base, uint32_t byteOff) {
    return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + byteOff);
}

constexpr int kDepth = 4;   // register slots of operand fragments (3 steps in flight + 1 in use)
// (the offsets are 32-bit: the host checks that one frequency plane stays below 2^32 bytes)

__global__ __launch_bounds__(kFusedThreads, 1) void wino_gemm_out_fused_kernel(const FusedParams p) {
    extern __shared__ __attribute__((aligned(16))) float Ml[];   // [64 f][16 k][32 t]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lrow = lane >> 5, lcol = lane & 31;

    // XCD-aware order: all output-channel blocks of one tile block run back to back on one XCD
    const int b = blockIdx.x, xcd = b & 7, j = b >> 3;
    const int tbl = j / p.nKB, kb = j - tbl * p.nKB;
    const int tb = tbl * 8 + xcd;
    if (tb >= p.nTB) return;

    // Per-frequency base pointers are wave-uniform (scalar registers); the lane's part of the
    // address is one 32-bit offset shared by all 16 frequencies.
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    const size_t planeU = (size_t)p.C_pad * p.K_pad, planeV = (size_t)p.C_pad * p.T_pad;
    const float *ub = p.U + (size_t)(wv * kFW) * planeU + (size_t)kb * 32;
    const float *vbase = p.V + (size_t)(wv * kFW) * planeV + (size_t)tb * 32;
    // byte offsets; the host checks that a frequency plane is below 2^32 bytes
    uint32_t offU = 4u * ((uint32_t)lrow * p.K_pad + lcol), offV = 4u * ((uint32_t)lrow * (uint32_t)p.T_pad + lcol);
    const uint32_t stepU = 8u * p.K_pad, stepV = 8u * (uint32_t)p.T_pad;

    floatx16 acc[kFW];
#pragma unroll
    for (int f = 0; f < kFW; f++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[f][i] = 0.f;

    float a[kDepth][kFW], bv[kDepth][kFW];
    const int nSteps = p.C_pad / 2;       // a multiple of kDepth: C_pad is a multiple of 8
#pragma unroll
    for (int d = 0; d < kDepth - 1; d++) {      // nSteps >= 4: no bounds test needed
#pragma unroll
        for (int f = 0; f < kFW; f++) {
            a[d][f] = ldg(ub + f * planeU, offU);
            bv[d][f] = ldg(vbase + f * planeV, offV);
        }
        offU += stepU;
        offV += stepV;
    }
    // Steady state: every step prefetches the step three ahead (no branches inside, so the
    // compiler's wait counts stay partial); the last four steps are peeled.
    for (int s0 = 0; s0 + kDepth < nSteps; s0 += kDepth) {
#pragma unroll
        for (int u = 0; u < kDepth; u++) {
            const int slot = (u + kDepth - 1) % kDepth;
#pragma unroll
            for (int f = 0; f < kFW; f++) {
                a[slot][f] = ldg(ub + f * planeU, offU);
                bv[slot][f] = ldg(vbase + f * planeV, offV);
            }
            offU += stepU;
            offV += stepV;
#pragma unroll
            for (int f = 0; f < kFW; f++)
                acc[f] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][f], bv[u][f], acc[f], 0, 0, 0);
        }
    }
    // last group: step nSteps-4 still prefetches step nSteps-1
#pragma unroll
    for (int f = 0; f < kFW; f++) {
        a[kDepth - 1][f] = ldg(ub + f * planeU, offU);
        bv[kDepth - 1][f] = ldg(vbase + f * planeV, offV);
    }
#pragma unroll
    for (int u = 0; u < kDepth; u++)
#pragma unroll
        for (int f = 0; f < kFW; f++)
            acc[f] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[u][f], bv[u][f], acc[f], 0, 0, 0);

    fused_output_transform(p.out, acc, Ml, kb, tb);
}

}  // namespace

extern "C" int fc_wino_gemm_output_fused(fc_context *ctx, const fc_wino_plan *plan, const float *U_dev,
                                         const float *V_dev, const float *bias_dev, int relu, float *y_dev) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !U_dev || !V_dev || !y_dev)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_output_fused: null argument", hipSuccess);
    fc_wino_plan chk;
    if (fc_wino_make_plan(&plan->shape, plan->gemm_config, &chk) != FC_OK || !fc_same_wino_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_output_fused: plan does not describe a supported layer", hipSuccess);
    if ((size_t)plan->C_pad * plan->T_pad >= (1ull << 30) || (size_t)plan->C_pad * plan->K_pad >= (1ull << 30))
        return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_gemm_output_fused: a frequency plane of U or V exceeds 4 GiB", hipSuccess);
    if (plan->K_pad % 32 || plan->T_pad % 32 || plan->C_pad % 8)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_output_fused: padded sizes must be multiples of 32 (K, T) and 8 (C)", hipSuccess);
    if (((uintptr_t)y_dev & 7) != 0)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_output_fused: y must be 8-byte aligned", hipSuccess);
    if (!ctx->fused_lds_granted) {
        if (ctx->capturing)
            return fc_set_error(ctx, FC_ERR_STATE, "fc_wino_gemm_output_fused: run this kernel once before recording a graph with it", hipSuccess);
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_gemm_out_fused_kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFusedLdsBytes));
        ctx->fused_lds_granted = true;
    }
    FusedParams p;
    p.U = U_dev; p.V = V_dev;
    p.out = make_fused_out(plan, bias_dev, relu, y_dev);
    p.K_pad = plan->K_pad; p.C_pad = plan->C_pad; p.T_pad = plan->T_pad;
    p.nKB = plan->K_pad / 32;
    p.nTB = (int)((plan->T + 31) / 32);
    const long tbGroups = (p.nTB + 7) / 8;
    const long blocks = tbGroups * 8 * p.nKB;
    if (blocks >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_gemm_output_fused: grid too large", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_FUSED_GEMM_OUT);
    wino_gemm_out_fused_kernel<<<dim3((unsigned)blocks), dim3(kFusedThreads), kFusedLdsBytes, ctx->stream>>>(p);
    FC_LAUNCH_CHECK(ctx, "wino_gemm_out_fused_kernel");
    return FC_OK;
}

extern "C" int fc_wino_prefer_fused(const fc_conv_shape *s) {
    if (!fc_shape_ok(s)) return 0;
    if ((long)s->C * s->K > 8192) return 0;
    if (s->C <= 8) return 1;      // next to no products: the output transform is all there is
    // one block of 32 tiles x 32 output channels per workgroup, one workgroup per CU at a time
    const long OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1), OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    const long blocks = ((long)s->N * ((OH + 5) / 6) * ((OW + 5) / 6) + 31) / 32 * ((s->K + 31) / 32);
    return blocks >= 512 ? 1 : 0;
}

extern "C" int fc_wino_forward_fused(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, const float *w_dev,
                                     const float *bias_dev, int relu, int filter_ready, float *U_dev, float *V_dev,
                                     float *y_dev) {
    const int rc = filter_ready ? fc_wino_input_transform(ctx, plan, x_dev, V_dev)
                                : fc_wino_filter_input_transform(ctx, plan, w_dev, U_dev, x_dev, V_dev);
    if (rc) return rc;
    return fc_wino_gemm_output_fused(ctx, plan, U_dev, V_dev, bias_dev, relu, y_dev);
}
