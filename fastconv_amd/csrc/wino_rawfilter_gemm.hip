// Winograd GEMM stage for layers with few tiles (batch 1 on small images), fed by the
// untransformed 3x3 filter instead of U.
//
// With T tiles a frequency-plane GEMM does 2*K*C*T flop on K*C operands of U: at T <= 32 the
// stage is a pass over U, which is 64/9 times the filter (67 MB for 512 -> 512 channels, written
// by the filter transform and read back here when the transform is online).  This kernel reads
// the 9 filter taps instead and forms U in registers: the A operand of v_mfma_f32_16x16x4_f32
// is one value per lane, A[row = lane % 16][depth = lane / 16], so a lane that holds the filter of
// (output channel kb*16 + lane % 16, one input channel per depth step) can make, for every
// frequency (i, j), exactly the operand the product of that frequency needs:
//     U_ij[k][c] = sum_b (sum_a G[i][a] g[k][c][a][b]) G[j][b].
// A workgroup covers 4*FPW frequencies of 16 output channels: at most two rows i.  The inner sum
// (three values per row i, filter and channel) is made once per group of four wavefronts, by the
// thread that fetched the filter, and handed over through LDS; a wavefront then spends 3*FPW
// multiply-adds per lane and depth step beside its FPW*NT MFMAs.  The workgroups of one block of
// 16 output channels sit on one XCD so that the filter is fetched into one L2.
#include "fc_internal.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct RawGemmParams {
    const float *w;      // [K][C][3][3]
    const float *V;      // [64][C_pad][T_pad]
    float *M;            // [64][K_pad][T_pad]
    int K, C, C_pad, K_pad, T_pad;
    int kBlocks8;        // blocks of 16 output channels, rounded up to a multiple of 8
    int tBlocks;         // blocks of 16*NT tiles
};

// rows of G (winoF63ZC/winoF63ZC.cpp:137-166)
__constant__ float kG[8][4] = {
    {1.f, 0.f, 0.f, 0.f},
    {(float)(-2.0 / 9), (float)(-2.0 / 9), (float)(-2.0 / 9), 0.f},
    {(float)(-2.0 / 9), (float)(2.0 / 9), (float)(-2.0 / 9), 0.f},
    {(float)(1.0 / 90), (float)(1.0 / 45), (float)(2.0 / 45), 0.f},
    {(float)(1.0 / 90), (float)(-1.0 / 45), (float)(2.0 / 45), 0.f},
    {(float)(1.0 / 45), (float)(1.0 / 90), (float)(1.0 / 180), 0.f},
    {(float)(1.0 / 45), (float)(-1.0 / 90), (float)(1.0 / 180), 0.f},
    {0.f, 0.f, 1.f, 0.f},
};

// One chunk = 16 input channels = 4 depth steps; in step m lane (r = lane % 16, d = lane / 16) multiplies
// channel c0 + 4*d + m.
//
// S: the input channels are split over S groups of four wavefronts (more wavefronts per SIMD to cover the
// latencies of a step: LDS round trip, barrier, dependent MFMAs); their sums meet in LDS at the end.
template <int FPW, int NT, int PF, int S>
__global__ __launch_bounds__(256 * S) void wino_rawfilter_gemm_kernel(const RawGemmParams p) {
    const int tid = threadIdx.x & 255, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int sp = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8);
    constexpr int FG = 16 / FPW;                 // frequency groups: 4*FPW frequencies per workgroup
    constexpr int IROWS = FPW == 4 ? 2 : 1;      // rows i a workgroup covers
    // blocks of one group of 16 output channels on one XCD (workgroups are dealt to the XCDs round robin)
    const uint32_t b = blockIdx.x, xcd = b & 7, idx = b >> 3;
    const uint32_t perKb = FG * p.tBlocks;
    const uint32_t kq = idx / perKb, rem = idx - kq * perKb;
    const uint32_t kb = kq * 8 + xcd;
    if ((int)(kb * 16) >= p.K) return;
    const uint32_t fg = rem / p.tBlocks, tb = rem - fg * p.tBlocks;
    const int fWg = (int)(fg * 4 * FPW);                                   // first frequency of the workgroup
    const int f0 = __builtin_amdgcn_readfirstlane(fWg + wave * FPW);      // of the wavefront
    const int iWg = fWg >> 3, iWave = (f0 >> 3) - iWg, fj = f0 & 7;
    float gi[IROWS][3];
#pragma unroll
    for (int ir = 0; ir < IROWS; ir++) {
        gi[ir][0] = kG[iWg + ir][0];
        gi[ir][1] = kG[iWg + ir][1];
        gi[ir][2] = kG[iWg + ir][2];
    }
    float gj[FPW][3];
#pragma unroll
    for (int q = 0; q < FPW; q++) {
        gj[q][0] = kG[fj + q][0];
        gj[q][1] = kG[fj + q][1];
        gj[q][2] = kG[fj + q][2];
    }

    const int r = lane & 15, d = lane >> 4;
    const int C = p.C;                                  // a multiple of 16
    // Every global address is a uniform base (scalar registers, advanced by addition) plus one 32-bit lane offset.
    //
    // Filter: thread (lk = tid / 16, lc = tid % 16) of a group fetches the 9 taps of output channel lk, channel
    // lc of the chunk (consecutive threads read consecutive 36-byte pieces), applies G from the left for the
    // rows i of the workgroup and stores 3 values per row to LDS, [row i][16 output channels][16 channels][3]
    // with the output channels 208 bytes apart: lane (r, d) reads the 12 values of its four channels as three
    // 16-byte pieces, and 16 lanes fall into different banks.
    constexpr int kKBytes = 208, kRowIBytes = 16 * kKBytes, kBufBytes = IROWS * kRowIBytes;
    extern __shared__ __attribute__((aligned(16))) char ldsAll[];      // [S][2][IROWS][16][208]
    char *lds = ldsAll + sp * (2 * kBufBytes);
    const int lk = tid >> 4, lc = tid & 15;
    const int krow = min((int)kb * 16 + lk, p.K - 1) - (int)kb * 16;      // rows past K repeat the last filter
    const uint32_t wOff = (uint32_t)((krow * C + lc) * 36);
    const uint32_t tWrite = (uint32_t)(lk * kKBytes + lc * 12);
    const uint32_t tRead = (uint32_t)(iWave * kRowIBytes + r * kKBytes + d * 48);
    const uint32_t planeV = (uint32_t)p.C_pad * p.T_pad;
    const uint32_t vOff = (uint32_t)((4 * d * p.T_pad + r) * 4);
    const size_t rowFloats = (size_t)p.T_pad;
    const int nChunks = C / 16 / S;                     // of this group
    const float *wNext = uniform_ptr(p.w + (size_t)kb * 16 * C * 9 + (size_t)sp * nChunks * (16 * 9));
    const float *vNext = uniform_ptr(p.V + (size_t)f0 * planeV + tb * (16 * NT) + (size_t)sp * nChunks * 16 * rowFloats);

    floatx4 acc[FPW][NT];
#pragma unroll
    for (int q = 0; q < FPW; q++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[q][nt] = floatx4{0.f, 0.f, 0.f, 0.f};

    // the next chunk: this thread's filter and FPW*NT*4 values of V.  Past the last chunk the pointers stop
    // advancing and the last chunk is read again, unused (no branch around loads: the compiler waits for every
    // load in flight where such paths join).
    int fetched = 0;
    auto load = [&](float (&g)[9], float (&bv)[FPW][NT][4]) {
        uint32_t wo = wOff, vo = vOff;
        asm volatile("" : "+v"(wo), "+v"(vo));      // keeps the widening of the offsets next to the loads
#pragma unroll
        for (int e = 0; e < 9; e++) g[e] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(wNext) + wo + e * 4);
        const float *bq = vNext;
#pragma unroll
        for (int q = 0; q < FPW; q++) {
            const float *bm = bq;
#pragma unroll
            for (int m = 0; m < 4; m++) {
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    bv[q][nt][m] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(bm) + vo + nt * 64);
                bm = uniform_ptr(bm + rowFloats);
            }
            bq = uniform_ptr(bq + planeV);
        }
        fetched++;
        const bool more = fetched < nChunks;
        wNext = uniform_ptr(wNext + (more ? 16 * 9 : 0));
        vNext = uniform_ptr(vNext + (more ? 16 * rowFloats : 0));
    };
    // G from the left, for the rows of the workgroup: t[b] = sum_a G[i][a] g[a][b]
    auto to_lds = [&](int buf, const float (&g)[9]) {
        char *dst = lds + buf * kBufBytes + tWrite;
#pragma unroll
        for (int ir = 0; ir < IROWS; ir++)
#pragma unroll
            for (int bb = 0; bb < 3; bb++)
                *reinterpret_cast<float *>(dst + ir * kRowIBytes + bb * 4) = gi[ir][0] * g[bb] + gi[ir][1] * g[3 + bb] + gi[ir][2] * g[6 + bb];
    };
    // G^T from the right, for the frequencies of the wavefront, and the products
    auto compute = [&](int buf, const float (&bv)[FPW][NT][4]) {
        floatx4 t[3];      // [m][b]
        const char *src = lds + buf * kBufBytes + tRead;
#pragma unroll
        for (int e = 0; e < 3; e++) t[e] = *reinterpret_cast<const floatx4 *>(src + e * 16);
        auto tf = [&](int e) { return t[e >> 2][e & 3]; };
#pragma unroll
        for (int m = 0; m < 4; m++) {
#pragma unroll
            for (int q = 0; q < FPW; q++) {
                const float u = tf(m * 3) * gj[q][0] + tf(m * 3 + 1) * gj[q][1] + tf(m * 3 + 2) * gj[q][2];
#pragma unroll
                for (int nt = 0; nt < NT; nt++)
                    acc[q][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(u, bv[q][nt][m], acc[q][nt], 0, 0, 0);
            }
        }
    };

    // PF register sets in flight; two LDS buffers, one barrier per chunk: the buffer written in step c was last
    // read in step c-2, and every wavefront has passed the barrier of step c-1 since.
    float ws[PF][9];
    float bs[PF][FPW][NT][4];
#pragma unroll
    for (int u = 0; u < PF; u++) load(ws[u], bs[u]);
    int ch = 0;
    for (; ch + PF <= nChunks; ch += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++) {
            const int buf = (ch + u) & 1;
            to_lds(buf, ws[u]);
            __syncthreads();
            compute(buf, bs[u]);
            load(ws[u], bs[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < PF - 1; u++)
        if (ch + u < nChunks) {
            const int buf = (ch + u) & 1;
            to_lds(buf, ws[u]);
            __syncthreads();
            compute(buf, bs[u]);
        }

    if (S > 1) {
        // sums of the groups: groups 1 .. S-1 leave theirs in LDS (the staging buffers are free now), group 0 adds
        floatx4 *red = reinterpret_cast<floatx4 *>(ldsAll);      // [S-1][256][FPW*NT]
        __syncthreads();
        if (sp > 0) {
#pragma unroll
            for (int q = 0; q < FPW; q++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) red[((sp - 1) * 256 + tid) * (FPW * NT) + q * NT + nt] = acc[q][nt];
        }
        __syncthreads();
        if (sp > 0) return;
#pragma unroll
        for (int o = 1; o < S; o++)
#pragma unroll
            for (int q = 0; q < FPW; q++)
#pragma unroll
                for (int nt = 0; nt < NT; nt++) acc[q][nt] += red[((o - 1) * 256 + tid) * (FPW * NT) + q * NT + nt];
    }

    // D[row = 4*d + e][col = r]
    const uint32_t planeM = (uint32_t)p.K_pad * p.T_pad;
    float *mq = uniform_ptr(p.M + (size_t)f0 * planeM + (size_t)kb * 16 * p.T_pad + tb * (16 * NT));
    const uint32_t mOff = (uint32_t)((4 * d * p.T_pad + r) * 4);
    bool rowInside[4];      // padding rows of M are written as zeros, as fc_wino_gemm leaves them
#pragma unroll
    for (int e = 0; e < 4; e++) rowInside[e] = (int)kb * 16 + 4 * d + e < p.K;
#pragma unroll
    for (int q = 0; q < FPW; q++) {
        float *me = mq;
#pragma unroll
        for (int e = 0; e < 4; e++) {
#pragma unroll
            for (int nt = 0; nt < NT; nt++)
                *reinterpret_cast<float *>(reinterpret_cast<char *>(me) + mOff + nt * 64) = rowInside[e] ? acc[q][nt][e] : 0.f;
            me = uniform_ptr(me + rowFloats);
        }
        mq = uniform_ptr(mq + planeM);
    }
}

// tiles a workgroup covers per frequency: 16 * NT
int raw_nt(long T) { return T <= 16 ? 1 : T <= 32 ? 2 : 4; }

}  // namespace

// The layers this path is for: few tiles and a filter that is large beside them.
extern "C" int fc_wino_raw_filter_gemm_applies(const fc_wino_plan *plan) {
    if (!plan) return 0;
    const fc_conv_shape &s = plan->shape;
    if (plan->T > 64 || s.C % 16 != 0) return 0;
    const int nt = raw_nt(plan->T);
    if (plan->T_pad % (16 * nt) != 0 || plan->K_pad % 16 != 0) return 0;
    if ((size_t)plan->C_pad * plan->T_pad >= (1u << 28) || (size_t)plan->K_pad * plan->T_pad >= (1u << 28)) return 0;
    if ((size_t)s.C * 16 * 36 >= (1u << 31)) return 0;
    return 1;
}

// Measured on MI355X at batch 1 (filter transform + fc_wino_gemm against this kernel, whole layer):
// 512 -> 512 channels at 7x7, 14x14 and 28x28 37 -> 28-31 us, 256 -> 512 at 28x28 29 -> 25, 256 -> 256 at
// 14x14 24 -> 19, 128 -> 128 at 28x28 level; with 49 tiles (256 -> 256 at 42x42) level.  Against
// fc_wino_gemm alone (filter transformed beforehand) the two are level at best: this is the path of
// the online strategy.
extern "C" int fc_wino_prefer_raw_filter_gemm(const fc_wino_plan *plan) {
    if (!fc_wino_raw_filter_gemm_applies(plan)) return 0;
    return plan->T <= 32 && (long)plan->shape.K * plan->shape.C >= 32768;
}

extern "C" int fc_wino_gemm_raw_filter(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev, const float *V_dev,
                                       float *M_dev, int freqs_per_wave, int channel_split) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !w_dev || !V_dev || !M_dev)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_raw_filter: null argument", hipSuccess);
    fc_wino_plan chk;
    if (fc_wino_make_plan(&plan->shape, plan->gemm_config, &chk) != FC_OK || !fc_same_wino_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_raw_filter: plan fields were modified after fc_wino_make_plan", hipSuccess);
    if (!fc_wino_raw_filter_gemm_applies(plan))
        return fc_set_error(ctx, FC_ERR_UNSUPPORTED,
                            "fc_wino_gemm_raw_filter: needs at most 64 tiles and a multiple of 16 input channels", hipSuccess);
    if (((uintptr_t)w_dev | (uintptr_t)V_dev | (uintptr_t)M_dev) & 15)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_raw_filter: buffers must be 16-byte aligned", hipSuccess);
    const fc_conv_shape &s = plan->shape;
    RawGemmParams p;
    p.w = w_dev; p.V = V_dev; p.M = M_dev;
    p.K = s.K; p.C = s.C; p.C_pad = plan->C_pad; p.K_pad = plan->K_pad; p.T_pad = (int)plan->T_pad;
    const int nt = raw_nt(plan->T);
    p.tBlocks = (int)((plan->T + 16 * nt - 1) / (16 * nt));
    const int kBlocks = (s.K + 15) / 16;
    p.kBlocks8 = (kBlocks + 7) / 8 * 8;
    // frequencies per wavefront: as many as still give every CU a workgroup
    int fpw = 4;
    while (fpw > 1 && (long)kBlocks * (16 / fpw) * p.tBlocks < 256) fpw /= 2;
    if (freqs_per_wave != 0) {
        if (freqs_per_wave != 1 && freqs_per_wave != 2 && freqs_per_wave != 4)
            return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_raw_filter: freqs_per_wave must be 0, 1, 2 or 4", hipSuccess);
        fpw = freqs_per_wave;
    }
    const long blocks = (long)p.kBlocks8 * (16 / fpw) * p.tBlocks;
    if (blocks >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_gemm_raw_filter: grid too large", hipSuccess);
    // groups of wavefronts over the input channels: two measure best (four are allowed where the registers of a
    // 1024-thread workgroup suffice, i.e. with one block of 16 tiles)
    const int splitMax = nt == 1 ? 4 : nt == 2 ? 2 : 1;
    int split = splitMax > 1 ? 2 : 1;
    while (split > 1 && (s.C / 16) % split) split /= 2;
    if (channel_split != 0) {
        if ((channel_split != 1 && channel_split != 2 && channel_split != 4) || channel_split > splitMax ||
            (s.C / 16) % channel_split)
            return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm_raw_filter: channel_split must be 0, 1, 2 or 4 and fit the layer", hipSuccess);
        split = channel_split;
    }
    fc_stage_scope scope(ctx, FC_STAGE_TENSOR_GEMM);
#define FC_RAW_LAUNCH(FPW_, NT_, S_)                                                                             \
    do {                                                                                                         \
        constexpr int PF_ = S_ == 4 && FPW_ * NT_ > 2 ? 2 : FPW_ * NT_ <= 4 ? 4 : FPW_ * NT_ <= 8 ? 3 : 2;      /* chunks in flight */ \
        constexpr size_t stage_ = (size_t)S_ * 2 * (FPW_ == 4 ? 2 : 1) * 16 * 208, red_ = (size_t)(S_ - 1) * 256 * FPW_ * NT_ * 16;     \
        wino_rawfilter_gemm_kernel<FPW_, NT_, PF_, S_>                                                           \
            <<<dim3((unsigned)blocks), dim3(256 * S_), stage_ > red_ ? stage_ : red_, ctx->stream>>>(p);         \
    } while (0)
#define FC_RAW_NT(FPW_)                                                       \
    do {                                                                      \
        if (nt == 1) {                                                        \
            if (split == 4) FC_RAW_LAUNCH(FPW_, 1, 4);                        \
            else if (split == 2) FC_RAW_LAUNCH(FPW_, 1, 2);                   \
            else FC_RAW_LAUNCH(FPW_, 1, 1);                                   \
        } else if (nt == 2) {                                                 \
            if (split == 2) FC_RAW_LAUNCH(FPW_, 2, 2);                        \
            else FC_RAW_LAUNCH(FPW_, 2, 1);                                   \
        } else FC_RAW_LAUNCH(FPW_, 4, 1);                                     \
    } while (0)
    if (fpw == 4) FC_RAW_NT(4);
    else if (fpw == 2) FC_RAW_NT(2);
    else FC_RAW_NT(1);
#undef FC_RAW_NT
#undef FC_RAW_LAUNCH
    FC_LAUNCH_CHECK(ctx, "wino_rawfilter_gemm_kernel");
    return FC_OK;
}
