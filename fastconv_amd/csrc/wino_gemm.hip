// Batched fp32 GEMM of the Winograd pipeline on gfx950 MFMA:
//   M[f][k][t] = sum_c U[f][c][k] * V[f][c][t]      f = 0..63, one launch.
// Both operands are stored reduction-index-major with the GEMM row/column index
// fastest, which is exactly the order v_mfma_f32_32x32x2_f32 wants its lanes in
// (lane l holds row/col l%32 of reduction step l/32), so tiles go global -> LDS
// as straight 16-byte copies and LDS -> registers as conflict-free dword reads.
#include <cmath>
#include <utility>

#include "fc_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// Copy passes written as pack expansions, so that every register-array index is a
// literal constant: with a loop index the arrays are not promoted to registers
// and the tile makes a round trip through scratch memory.
// `base` is the same for the whole workgroup (it stays in scalar registers); a lane adds its
// 32-bit byte offset: no vector instruction goes into the addresses.
template <int... I>
__device__ __forceinline__ void load_rows(floatx4 (&r)[sizeof...(I)], const float *base, uint32_t laneOff, size_t rowStride,
                                          std::integer_sequence<int, I...>) {
    // row after row by addition: pinned operands keep the sums in the scalar unit.  The empty asm keeps the widening of
    // the lane offset next to the loads (hoisted out of a loop it turns each address into a 64-bit vector sum)
    asm volatile("" : "+v"(laneOff));
    const float *b = uniform_ptr(base);
    ((r[I] = *reinterpret_cast<const floatx4 *>(reinterpret_cast<const char *>(b) + laneOff), b = uniform_ptr(b + rowStride)), ...);
}
template <int... I>
__device__ __forceinline__ void store_rows(float *lds, const floatx4 (&r)[sizeof...(I)], int rowStride,
                                           std::integer_sequence<int, I...>) {
    ((*reinterpret_cast<floatx4 *>(lds + I * rowStride) = r[I]), ...);
}

// Stages s0 .. s0+PF-1 with their register set as a compile-time constant.
template <class F, int... U>
__device__ __forceinline__ void stage_group(F &stage, int s0, std::integer_sequence<int, U...>) {
    (stage(s0 + U, std::integral_constant<int, U>()), ...);
}
template <class F, int... U>
__device__ __forceinline__ void stage_rest(F &stage, int s0, int nStages, std::integer_sequence<int, U...>) {
    ((s0 + U < nStages ? stage(s0 + U, std::integral_constant<int, U>()) : (void)0), ...);
}

// Workgroup tile BM x BN x BK; WGM x WGN wavefronts, each owning
// (BM/WGM) x (BN/WGN) of the tile as 32x32 MFMA blocks.
template <int BM, int BN, int BK, int WGM, int WGN>
struct GemmTile {
    static constexpr int THREADS = 64 * WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int A_VEC = BK * BM / 4, B_VEC = BK * BN / 4;      // float4 per stage
    static constexpr int A_LD = A_VEC / THREADS, B_LD = B_VEC / THREADS;
    static constexpr int A_ROWS = THREADS * 4 / BM, B_ROWS = THREADS * 4 / BN;   // tile rows per copy pass
    static constexpr int LDS_BYTES = 2 * BK * (BM + BN) * 4;
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be whole 32x32 MFMA blocks");
    static_assert(BK % 4 == 0, "fragments are fetched for two 32x32x2 MFMA steps at a time");
    static_assert(A_VEC % THREADS == 0 && B_VEC % THREADS == 0, "every thread copies the same number of float4");
    static_assert(A_LD >= 1 && B_LD >= 1, "tile smaller than one copy pass");
};

// One workgroup tile: M[f][kb*BM .. +BM][tb*BN .. +BN] = sum over all input channels.
// `smem` holds the two LDS stages of both operands (2*BK*(BM+BN) floats).
template <class TL>
__device__ __forceinline__ void gemm_tile(const float *__restrict__ U, const float *__restrict__ V,
                                          float *__restrict__ M, int K_pad, int C_pad, int T_pad, int f, int kb,
                                          int tb, float *smem) {
    constexpr int BM = TL::BM_, BN = TL::BN_, BK = TL::BK_;
    constexpr int MI = TL::MI, NI = TL::NI, A_LD = TL::A_LD, B_LD = TL::B_LD;
    // LDS: A stages 0 and 1, then B stages 0 and 1
    float *const As0 = smem, *const Bs0 = smem + 2 * BK * BM;

    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm0 = (wave / TL::WGN_) * TL::WM, wn0 = (wave % TL::WGN_) * TL::WN;

    // this thread's float4 of each copy pass: row r0 + i*ROWS, column c4
    const int arow = tid / (BM / 4), acol = (tid % (BM / 4)) * 4;
    const int brow = tid / (BN / 4), bcol = (tid % (BN / 4)) * 4;
    // global tiles: a uniform base per operand and stage, and one byte offset per lane (at most 8 rows of K_pad or
    // T_pad floats: the host checks that a row of either fits 2^28 floats)
    const float *ag = U + (size_t)f * C_pad * K_pad + (size_t)kb * BM;
    const float *bg = V + (size_t)f * C_pad * T_pad + (size_t)tb * BN;
    const uint32_t aOff = 4u * ((uint32_t)arow * (uint32_t)K_pad + acol), bOff = 4u * ((uint32_t)brow * (uint32_t)T_pad + bcol);
    const size_t aStage = (size_t)BK * K_pad, bStage = (size_t)BK * T_pad;
    const int aLds = arow * BM + acol, bLds = brow * BN + bcol;

    using SeqA = std::make_integer_sequence<int, A_LD>;
    using SeqB = std::make_integer_sequence<int, B_LD>;
    const size_t aPass = (size_t)TL::A_ROWS * K_pad, bPass = (size_t)TL::B_ROWS * T_pad;
    // Register set u holds the stages s with s % PF == u: a stage is fetched PF stages before
    // it is parked in LDS, which is what covers the latency of L2 and HBM when a stage holds
    // only a few MFMAs per wavefront.
    constexpr int PF = TL::PF_;
    const int nStages = C_pad / BK;
    floatx4 ra[PF][A_LD], rb[PF][B_LD];
#pragma unroll
    for (int u = 0; u < PF; u++)
        if (u < nStages) {
            load_rows(ra[u], ag + (size_t)u * aStage, aOff, aPass, SeqA());
            load_rows(rb[u], bg + (size_t)u * bStage, bOff, bPass, SeqB());
        }

    floatx16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < NI; ni++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mi][ni][i] = 0.f;

    store_rows(As0 + aLds, ra[0], TL::A_ROWS * BM, SeqA());
    store_rows(Bs0 + bLds, rb[0], TL::B_ROWS * BN, SeqB());
    if (PF < nStages) {
        load_rows(ra[0], ag + (size_t)PF * aStage, aOff, aPass, SeqA());
        load_rows(rb[0], bg + (size_t)PF * bStage, bOff, bPass, SeqB());
    }
    // the stage the loop fetches next: stage 1 + PF, advanced by one stage per fetch
    const float *agNext = uniform_ptr(ag + (size_t)(1 + PF) * aStage), *bgNext = uniform_ptr(bg + (size_t)(1 + PF) * bStage);
    __syncthreads();

    // fragment addresses: lane l reads element (row kk + l/32, column base + l%32)
    const int lrow = lane >> 5, lcol = lane & 31;
    const int aFrag = lrow * BM + wm0 + lcol, bFrag = lrow * BN + wn0 + lcol;
    // one stage: MFMAs out of LDS buffer s % 2; half way through, stage s+1 moves from register
    // set (u+1) % PF into the other buffer and that set is refilled with stage s+1+PF
    auto stage = [&](const int s, auto uc) __attribute__((always_inline)) {
        constexpr int u = decltype(uc)::value;
        const int buf = s & 1;
        const float *as = As0 + buf * (BK * BM), *bs = Bs0 + buf * (BK * BN);
        const bool more = s + 1 < nStages;
        constexpr int un = (u + 1) % PF;
        // Fragments are fetched two reduction steps (kk, kk+2) at a time, a pair ahead of the MFMAs that use them.
        // The two reads of a pair are 2*BM (2*BN) floats apart, a multiple of 64 dwords: one ds_read2st64 with both
        // offsets as immediates off the stage's base register, where a pair of neighbouring 32-wide blocks needed
        // a vector add per step for its address.
        // (one base register per 32-wide block, made opaque: seen as base + 32 dwords the compiler pairs
        // neighbouring blocks again)
        typedef const __attribute__((address_space(3))) float *LdsPtr;
        LdsPtr asb[MI], bsb[NI];
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            asb[mi] = (LdsPtr)(as + aFrag + mi * 32);
            asm volatile("" : "+v"(asb[mi]));
        }
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            bsb[ni] = (LdsPtr)(bs + bFrag + ni * 32);
            asm volatile("" : "+v"(bsb[ni]));
        }
        float a[2][2][MI], bb[2][2][NI];
#pragma unroll
        for (int mi = 0; mi < MI; mi++) {
            a[0][0][mi] = asb[mi][0];
            a[0][1][mi] = asb[mi][2 * BM];
        }
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            bb[0][0][ni] = bsb[ni][0];
            bb[0][1][ni] = bsb[ni][2 * BN];
        }
#pragma unroll
        for (int kq = 0; kq < BK / 4; kq++) {
            const int cur = kq & 1, nxt = cur ^ 1;
            if (kq + 1 < BK / 4) {
#pragma unroll
                for (int mi = 0; mi < MI; mi++) {
                    a[nxt][0][mi] = asb[mi][(4 * kq + 4) * BM];
                    a[nxt][1][mi] = asb[mi][(4 * kq + 6) * BM];
                }
#pragma unroll
                for (int ni = 0; ni < NI; ni++) {
                    bb[nxt][0][ni] = bsb[ni][(4 * kq + 4) * BN];
                    bb[nxt][1][ni] = bsb[ni][(4 * kq + 6) * BN];
                }
            }
            // the reads of the next pair are issued before the MFMAs of this one (the scheduler would put them behind)
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int st = 0; st < 2; st++)
#pragma unroll
                for (int mi = 0; mi < MI; mi++)
#pragma unroll
                    for (int ni = 0; ni < NI; ni++)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[cur][st][mi], bb[cur][st][ni], acc[mi][ni], 0, 0, 0);
            if (4 * kq == BK / 2 && more) {
                // the next stage goes to the other LDS buffer half way through this one's MFMAs,
                // and its registers are refilled with the stage PF further on
                store_rows(As0 + (buf ^ 1) * (BK * BM) + aLds, ra[un], TL::A_ROWS * BM, SeqA());
                store_rows(Bs0 + (buf ^ 1) * (BK * BN) + bLds, rb[un], TL::B_ROWS * BN, SeqB());
                if (s + 1 + PF < nStages) {
                    load_rows(ra[un], agNext, aOff, aPass, SeqA());
                    load_rows(rb[un], bgNext, bOff, bPass, SeqB());
                    agNext = uniform_ptr(agNext + aStage);
                    bgNext = uniform_ptr(bgNext + bStage);
                }
            }
        }
        __syncthreads();
    };
    int s0 = 0;
    for (; s0 + PF <= nStages; s0 += PF) stage_group(stage, s0, std::make_integer_sequence<int, PF>());
    // the last nStages % PF stages
    stage_rest(stage, s0, nStages, std::make_integer_sequence<int, PF - 1>());

    // D block layout: register i of lane l is row 8*(i/4) + 4*(l/32) + i%4, column l%32.
    // The wavefront's block starts at a uniform address; the lane's share of it (4 * lrow rows down, lcol columns in) is one byte offset.
    float *Mg = (M + ((size_t)f * K_pad + (size_t)kb * BM + wm0) * T_pad + (size_t)tb * BN + wn0);
    const uint32_t mOff = 4u * (4u * (uint32_t)lrow * (uint32_t)T_pad + lcol);
    const size_t rowBytes = (size_t)T_pad * 4;
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            // rows 0-3, 8-11, 16-19, 24-27 of the 32x32 block, stepped by addition in the scalar unit
            char *pr = reinterpret_cast<char *>(uniform_ptr(Mg + (size_t)(mi * 32) * T_pad + ni * 32));
#pragma unroll
            for (int i = 0; i < 16; i++) {
                *reinterpret_cast<float *>(pr + mOff) = acc[mi][ni][i];
                pr = uniform_ptr(pr + ((i % 4) == 3 ? 5 * rowBytes : rowBytes));
            }
        }
}

// Workgroups are dealt to the 8 XCDs round-robin by linear id.  All tiles of one
// frequency share U[f] and re-read V[f] once per output-channel block, so a
// frequency is kept on one XCD (one L2): tile id b -> xcd = b % 8, and the b / 8
// sequence walks that XCD's 8 frequencies one after another, output channel
// blocks innermost.
__device__ __forceinline__ void decode_tile(int b, int nKB, int nTB, int *f, int *kb, int *tb) {
    const int xcd = b & 7, idx = b >> 3;
    const int bpf = nKB * nTB;
    const int fl = idx / bpf, rem = idx - fl * bpf;
    *f = fl * 8 + xcd;
    *tb = rem / nKB;
    *kb = rem - *tb * nKB;
}

template <class TL>
__global__ __launch_bounds__(TL::THREADS) void wino_gemm_kernel(const float *__restrict__ U,
                                                                const float *__restrict__ V,
                                                                float *__restrict__ M, int K_pad, int C_pad,
                                                                int T_pad, int nKB, int nTB) {
    __shared__ __attribute__((aligned(16))) float smem[2 * TL::BK_ * (TL::BM_ + TL::BN_)];
    int f, kb, tb;
    decode_tile(blockIdx.x, nKB, nTB, &f, &kb, &tb);
    gemm_tile<TL>(U, V, M, K_pad, C_pad, T_pad, f, kb, tb, smem);
}

// Same product, with the last `nTiles - nBig` tiles of the grid cut into quarters, so
// that the tail of the grid (fewer tiles left than workgroup slots) still spreads over
// all compute units.  Worth 2-3 % on a 3200-tile layer; the time of this kernel is
// otherwise linear in the tile count (no visible rounds).
template <class BIG, class SMALL>
__global__ __launch_bounds__(BIG::THREADS) void wino_gemm_tail_kernel(const float *__restrict__ U,
                                                                      const float *__restrict__ V,
                                                                      float *__restrict__ M, int K_pad, int C_pad,
                                                                      int T_pad, int nKB, int nTB, int nBig) {
    static_assert(BIG::THREADS == SMALL::THREADS && BIG::BK_ == SMALL::BK_, "one launch shape for both tile sizes");
    static_assert(BIG::BM_ == 2 * SMALL::BM_ && BIG::BN_ == 2 * SMALL::BN_, "a big tile is four small tiles");
    __shared__ __attribute__((aligned(16))) float smem[2 * BIG::BK_ * (BIG::BM_ + BIG::BN_)];
    const int b = blockIdx.x;
    int f, kb, tb;
    if (b < nBig) {
        decode_tile(b, nKB, nTB, &f, &kb, &tb);
        gemm_tile<BIG>(U, V, M, K_pad, C_pad, T_pad, f, kb, tb, smem);
    } else {
        const int p = b - nBig, q = p & 3;
        decode_tile(nBig + (p >> 2), nKB, nTB, &f, &kb, &tb);
        gemm_tile<SMALL>(U, V, M, K_pad, C_pad, T_pad, f, 2 * kb + (q >> 1), 2 * tb + (q & 1), smem);
    }
}

// PF = register sets of global prefetch.  Measured on MI355X: 2 or 4 sets change the rate of the
// 64x64 tile by -2..+4 % depending on the layer and cost the larger tiles a resident workgroup
// (their register count nearly doubles), so every configuration runs with one.
template <int BM, int BN, int BK, int WGM, int WGN, int PF = 1>
struct TileCfg : GemmTile<BM, BN, BK, WGM, WGN> {
    static constexpr int BM_ = BM, BN_ = BN, BK_ = BK, WGM_ = WGM, WGN_ = WGN, PF_ = PF;
};

typedef TileCfg<128, 128, 16, 2, 2> Cfg0;
typedef TileCfg<64, 128, 16, 1, 2> Cfg1;
typedef TileCfg<128, 64, 16, 2, 1> Cfg2;
typedef TileCfg<64, 64, 16, 2, 2> Cfg3;
typedef TileCfg<32, 32, 16, 1, 1> Cfg4;
typedef TileCfg<128, 128, 8, 2, 2> Cfg5;
typedef TileCfg<64, 128, 8, 1, 2> Cfg6;
typedef TileCfg<256, 128, 16, 2, 2> Cfg7;
typedef TileCfg<128, 256, 16, 2, 2> Cfg8;
typedef TileCfg<128, 128, 32, 2, 2> Cfg9;
typedef TileCfg<64, 32, 16, 2, 1> Cfg10;

const fc_gemm_config kConfigs[] = {
#define FC_CFG(id, T) {id, T::BM_, T::BN_, T::BK_, T::WGM_, T::WGN_, T::LDS_BYTES, 1}
    FC_CFG(0, Cfg0), FC_CFG(1, Cfg1), FC_CFG(2, Cfg2), FC_CFG(3, Cfg3), FC_CFG(4, Cfg4), FC_CFG(5, Cfg5),
    FC_CFG(6, Cfg6), FC_CFG(7, Cfg7), FC_CFG(8, Cfg8), FC_CFG(9, Cfg9), FC_CFG(10, Cfg10),
#undef FC_CFG
};
const int kNumConfigs = sizeof(kConfigs) / sizeof(kConfigs[0]);

template <class TL>
void launch(fc_context *ctx, const fc_wino_plan *plan, const float *U, const float *V, float *M) {
    const int nKB = plan->K_pad / TL::BM_, nTB = (int)(plan->T_pad / TL::BN_);
    const dim3 grid(64u * nKB * nTB);
    wino_gemm_kernel<TL><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(U, V, M, plan->K_pad, plan->C_pad,
                                                                      (int)plan->T_pad, nKB, nTB);
}

// Tiles of the last, partly filled round that are worth quartering: none unless that
// round would be less than half full.  `slots` = workgroups resident at once.
long tail_tiles(long nTiles, long slots) {
    const long r = nTiles % slots;
    return (nTiles > slots && r > 0 && 2 * r <= slots) ? r : 0;
}

template <class BIG, class SMALL>
void launch_with_tail(fc_context *ctx, const fc_wino_plan *plan, const float *U, const float *V, float *M) {
    const int nKB = plan->K_pad / BIG::BM_, nTB = (int)(plan->T_pad / BIG::BN_);
    const long nTiles = 64l * nKB * nTB;
    const long slots = (long)ctx->props.multiProcessorCount * 4;      // 4 workgroups of this kernel fit one CU
    const long r = tail_tiles(nTiles, slots);
    if (r == 0) {
        launch<BIG>(ctx, plan, U, V, M);
        return;
    }
    const long nBig = nTiles - r;
    const dim3 grid((unsigned)(nBig + 4 * r));
    wino_gemm_tail_kernel<BIG, SMALL><<<grid, dim3(BIG::THREADS), 0, ctx->stream>>>(
        U, V, M, plan->K_pad, plan->C_pad, (int)plan->T_pad, nKB, nTB, (int)nBig);
}

}  // namespace

extern "C" int fc_wino_gemm_num_configs(void) { return kNumConfigs; }

extern "C" int fc_wino_gemm_get_config(int id, fc_gemm_config *cfg) {
    if (!cfg || id < 0 || id >= kNumConfigs) return FC_ERR_INVALID;
    *cfg = kConfigs[id];
    return FC_OK;
}

// Cost model behind the untuned choice: padded multiply-adds, divided by a rate per tile shape
// relative to 128x128x16 and by how evenly the grid fills the workgroup slots of the chip.  The
// rates start from what each shape sustains on a large layer (256 -> 256 channels at 56x56,
// batch 128) and are set so that the model picks a shape within 2 % of the best measured one on
// fifteen VGG-16 / ResNet-50 layers at batch 1, 32 and 128: in practice 128x128 for large grids,
// 64x64 for mid-sized ones (it loses less to padding and to uneven placement than its large-layer
// rate suggests), 32x32 where a 64-wide tile would be mostly padding.
extern "C" int fc_wino_gemm_default_config(const fc_conv_shape *s) {
    if (!fc_shape_ok(s)) return FC_ERR_INVALID;
    static const double kRate[] = {1.00, 0.90, 0.90, 0.97, 0.72, 0.95, 0.88, 0.93, 0.93, 0.90, 0.76};
    static_assert(sizeof(kRate) / sizeof(kRate[0]) == sizeof(kConfigs) / sizeof(kConfigs[0]), "one rate per configuration");
    const int OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1), OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    const double T = (double)s->N * ((OH + 5) / 6) * ((OW + 5) / 6);
    int best = 0;
    double bestCost = 1e300;
    for (int id = 0; id < kNumConfigs; id++) {
        const fc_gemm_config &c = kConfigs[id];
        const double kp = ceil((double)s->K / c.bm) * c.bm, tp = ceil(T / c.bn) * c.bn;
        const double cp = ceil((double)s->C / c.bk) * c.bk;
        const double blocks = 64.0 * (kp / c.bm) * (tp / c.bn);
        const double slots = 256.0 * (c.bm * c.bn > 128 * 128 || c.bk == 32 ? 2 : 4);
        // the time of a launch is nearly linear in its tile count: a partly filled last round costs
        // little, and nothing for configuration 0, whose last round runs as quartered tiles
        double fill = blocks / (ceil(blocks / slots) * slots);
        if (id == 0 && blocks > slots) fill = 1.0;
        const double cost = kp * tp * cp / (kRate[id] * (0.8 + 0.2 * fill));
        if (cost < bestCost) { bestCost = cost; best = id; }
    }
    return best;
}

extern "C" int fc_wino_gemm(fc_context *ctx, const fc_wino_plan *plan, const float *U_dev, const float *V_dev,
                            float *M_dev) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !U_dev || !V_dev || !M_dev) return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: null argument", hipSuccess);
    fc_gemm_config cfg;
    if (fc_wino_gemm_get_config(plan->gemm_config, &cfg)) return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: unknown tile configuration", hipSuccess);
    fc_wino_plan chk;
    if (fc_wino_make_plan(&plan->shape, plan->gemm_config, &chk) != FC_OK || !fc_same_wino_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: plan fields were modified after fc_wino_make_plan", hipSuccess);
    // the kernel has no edge predication: the buffers must be padded to the tile
    if (plan->K_pad <= 0 || plan->C_pad <= 0 || plan->T_pad <= 0 || plan->K_pad % cfg.bm || plan->C_pad % cfg.bk ||
        plan->T_pad % cfg.bn)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: padded sizes are not multiples of the tile", hipSuccess);
    const long blocks = 64l * (plan->K_pad / cfg.bm) * (plan->T_pad / cfg.bn);
    if (blocks >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_gemm: grid too large", hipSuccess);
    if (((uintptr_t)U_dev | (uintptr_t)V_dev | (uintptr_t)M_dev) & 15)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: buffers must be 16-byte aligned", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_TENSOR_GEMM);
    switch (plan->gemm_config) {
        case 0: launch_with_tail<Cfg0, Cfg3>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 1: launch<Cfg1>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 2: launch<Cfg2>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 3: launch<Cfg3>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 4: launch<Cfg4>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 5: launch<Cfg5>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 6: launch<Cfg6>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 7: launch<Cfg7>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 8: launch<Cfg8>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 9: launch<Cfg9>(ctx, plan, U_dev, V_dev, M_dev); break;
        case 10: launch<Cfg10>(ctx, plan, U_dev, V_dev, M_dev); break;
        default: return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_gemm: unknown tile configuration", hipSuccess);
    }
    FC_LAUNCH_CHECK(ctx, "wino_gemm_kernel");
    return FC_OK;
}
