// Implicit-GEMM convolution on gfx950 fp32 MFMA:
//   y[n][k][oh][ow] = sum_{c,r,s} w[k][c][r][s] * x[n][c][oh*sh + r - pt][ow*sw + s - pl]
// seen as D[K][N*OH*OW] = Wp^T[K][Kred] * col[Kred][N*OH*OW], where the column
// matrix is never written to memory: each workgroup gathers its BK x BN slice of
// it straight into LDS.  The filter is re-laid once to Wp[Kred_pad][K_pad]
// (output channel fastest) so that its tiles are straight 16-byte copies, as in
// the Winograd GEMM.
#include <cmath>
#include <cstdio>
#include <mutex>
#include <utility>

#include "fc_internal.h"

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));   // native vector: arrays of it stay in registers

// Order of the reduction index.  Channel-major (the column-matrix rows of
// convLayer/im2colConv.cpp:285-309): kred = (c*kh + r)*kw + s.  Tap-major, used whenever the channel
// count is a whole number of LDS stages (C % BK == 0): kred = (r*kw + s)*C + c, so that the BK rows of a
// stage share one filter tap -- one in-image test and one window offset per stage instead of one per
// gathered element, and consecutive rows are consecutive channels (no table lookups in the loop).
// The packed filter and the row table follow whichever order the layer uses.
// Row table entry for reduction row kred (tap (r, s) of channel c):
//   [2*kred]   = c*H*W + r*W + s      (offset from the window origin)
//   [2*kred+1] = r << 16 | s          (31 << 16 | 31 for padding rows: a mask bit that is never set)
__global__ __launch_bounds__(256) void igemm_pack_filter_kernel(const float *__restrict__ w,
                                                                float *__restrict__ Wp,
                                                                int32_t *__restrict__ table, int K, int C,
                                                                int kh, int kw, int H, int W, int Kred,
                                                                int Kred_pad, int K_pad, int tapMajor) {
    const int k = blockIdx.x * 64 + (threadIdx.x & 63);
    const int kred = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (kred >= Kred_pad) return;
    int c = 0, r = 31, s = 31;
    if (kred < Kred) {
        if (tapMajor) {
            const int t = kred / C;
            c = kred - t * C;
            r = t / kw;
            s = t - r * kw;
        } else {
            c = kred / (kh * kw);
            const int rs = kred - c * kh * kw;
            r = rs / kw;
            s = rs - r * kw;
        }
    }
    if (k < K_pad)
        Wp[(size_t)kred * K_pad + k] = (k < K && kred < Kred) ? w[((size_t)k * C + c) * (kh * kw) + r * kw + s] : 0.f;
    if (blockIdx.x == 0 && (threadIdx.x & 63) == 0) {
        table[2 * kred] = kred < Kred ? c * H * W + r * W + s : 0;
        table[2 * kred + 1] = (r << 16) | s;
    }
}

struct IgemmParams {
    const float *x;
    const float *Wp;
    const int32_t *table;
    const float *bias;
    float *y;
    int N, C, H, W, K, OH, OW, kh, kw, sh, sw, pt, pl, relu;
    int Kred_pad, K_pad;
    long Npix;
    int nKB, nPB;
    int splitK, stagesPerSplit;   // reduction split over blockIdx.y; partial sums go to ws
    float *ws;                    // [splitK][K][Npix] when splitK > 1
    long xBytes;                  // size of the input tensor
    int fastStore;                // K is a whole number of tiles, every output byte offset fits 32 bits, bias 16-byte aligned
    fc_fastdiv divOHW, divOW;
};

template <int BM, int BN, int BK, int WGM, int WGN>
struct IgTile {
    static constexpr int BM_ = BM, BN_ = BN, BK_ = BK, WGM_ = WGM, WGN_ = WGN;
    static constexpr int THREADS = 64 * WGM * WGN;
    static constexpr int WM = BM / WGM, WN = BN / WGN;
    static constexpr int MI = WM / 32, NI = WN / 32;
    static constexpr int A_VEC = BK * BM / 4;
    static constexpr int A_LD = A_VEC / THREADS;
    static constexpr int A_ROWS = THREADS * 4 / BM;     // filter-tile rows per copy pass
    static constexpr int ROW_STEP = THREADS / BN;       // gather: one column, every ROW_STEP-th row
    static constexpr int B_LD = BK / ROW_STEP;
    static constexpr int LDS_BYTES = 2 * BK * (BM + BN) * 4;
    // wavefronts per SIMD the register allocation must leave room for (the second argument of
    // __launch_bounds__ in HIP): four for the four-wavefront tiles up to 128x128 and 64x256
    static constexpr int MIN_WAVES = (BM * BN <= 128 * 128 && WGM * WGN == 4) ? 4 : 1;
    static_assert(THREADS % BN == 0 && BK % ROW_STEP == 0, "gather mapping");
    static_assert(BN % 64 == 0, "a wavefront gathers one row of the column matrix");
    static_assert(A_VEC % THREADS == 0 && A_LD >= 1, "every thread copies the same number of float4");
    static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be whole 32x32 MFMA blocks");
};

// Copy passes as pack expansions (literal register-array indices, see wino_gemm.hip).
template <int... I>
__device__ __forceinline__ void ig_load_rows(floatx4 (&r)[sizeof...(I)], const float *p, size_t rowStride,
                                             std::integer_sequence<int, I...>) {
    ((r[I] = *reinterpret_cast<const floatx4 *>(p + (size_t)I * rowStride)), ...);
}
// The same from a base all lanes share (scalar registers) and one 32-bit byte offset per lane: no vector
// instruction goes into the addresses (see load_rows in wino_gemm.hip).
template <int... I>
__device__ __forceinline__ void ig_load_rows_at(floatx4 (&r)[sizeof...(I)], const float *base, uint32_t laneOff, size_t rowStride,
                                                std::integer_sequence<int, I...>) {
    asm volatile("" : "+v"(laneOff));
    const float *b = uniform_ptr(base);
    ((r[I] = *reinterpret_cast<const floatx4 *>(reinterpret_cast<const char *>(b) + laneOff), b = uniform_ptr(b + rowStride)), ...);
}
template <int... I>
__device__ __forceinline__ void ig_store_rows(float *lds, const floatx4 (&r)[sizeof...(I)], int rowStride,
                                              std::integer_sequence<int, I...>) {
    ((*reinterpret_cast<floatx4 *>(lds + I * rowStride) = r[I]), ...);
}

// One gathered element of the column matrix.  The row (reduction index) is the same
// for the whole wavefront, so its table entry lives in scalar registers; the
// per-pixel part of the bounds test is two bit masks computed once per thread.
// The load is unconditional (an element outside the image reads the start of the image
// instead) and its value is not touched here: whether it counts is recorded as bit `slot`
// of `okBits` and applied when the element is written to LDS, so that the loads of a
// stage stay in flight under the MFMAs of the stage before.
// MASKED = false: no test at all (kept for completeness; the buffer modes below serve such layers).
template <bool MASKED>
__device__ __forceinline__ float ig_gather(const float *ximg, int pixOff, uint32_t maskR, uint32_t maskS,
                                           const int32_t *table, int kred, int slot, uint32_t &okBits) {
    const int off = table[2 * kred];
    if (!MASKED) return ximg[pixOff + off];
    const int rs = table[2 * kred + 1];
    const bool ok = ((maskR >> (rs >> 16)) & (maskS >> (rs & 0xffff)) & 1u) != 0;
    okBits |= ok ? (1u << slot) : 0u;
    return ximg[ok ? pixOff + off : 0];
}
template <bool MASKED, int... I>
__device__ __forceinline__ uint32_t ig_gather_rows(float (&r)[sizeof...(I)], const float *ximg, int pixOff,
                                                   uint32_t maskR, uint32_t maskS, const int32_t *table, int kred0,
                                                   int rowStep, std::integer_sequence<int, I...>) {
    uint32_t okBits = 0;
    ((r[I] = ig_gather<MASKED>(ximg, pixOff, maskR, maskS, table, kred0 + I * rowStep, I, okBits)), ...);
    return okBits;
}
template <bool MASKED, int... I>
__device__ __forceinline__ void ig_scatter_rows(float *lds, const float (&r)[sizeof...(I)], uint32_t okBits, int rowStride,
                                                std::integer_sequence<int, I...>) {
    ((lds[I * rowStride] = (!MASKED || ((okBits >> I) & 1u)) ? r[I] : 0.f), ...);
}

// The same element through a buffer resource over the whole input tensor (tensors below 2 GiB): the
// address is one 32-bit byte offset from a scalar base, and a tap outside the image gets bit 31 of
// its offset set, which puts it past the end of the buffer: the hardware's range check returns 0
// for it without touching memory.  No 64-bit address arithmetic, no select at the LDS write.
// invLo / invHi: bit t = r*kw + s is set when tap (r, s) of this thread's pixel lies outside the
// image (taps 64 and up, which only padding rows of the reduction name, count as outside).
template <bool MASKED>
__device__ __forceinline__ float ig_gather_buf(__amdgpu_buffer_rsrc_t xres, uint32_t pixByte, uint32_t invLo, uint32_t invHi,
                                               const int32_t *table, int kred, int kw) {
    uint32_t voff = pixByte + 4u * (uint32_t)table[2 * kred];
    if (MASKED) {
        const int rs = table[2 * kred + 1];
        const uint32_t t = (uint32_t)(rs >> 16) * (uint32_t)kw + (uint32_t)(rs & 0xffff);     // wave-uniform
        const uint32_t word = t < 32u ? invLo : invHi;
        const uint32_t bad = t < 64u ? (word >> (t & 31u)) & 1u : 1u;
        voff |= bad << 31;
    }
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xres, voff, 0, 0));
}
template <bool MASKED, int... I>
__device__ __forceinline__ void ig_gather_rows_buf(float (&r)[sizeof...(I)], __amdgpu_buffer_rsrc_t xres, uint32_t pixByte,
                                                   uint32_t invLo, uint32_t invHi, const int32_t *table, int kred0, int rowStep,
                                                   int kw, std::integer_sequence<int, I...>) {
    ((r[I] = ig_gather_buf<MASKED>(xres, pixByte, invLo, invHi, table, kred0 + I * rowStep, kw)), ...);
}

// How the B tile (a slice of the column matrix) reaches LDS.  IG_GATHER is the fallback of the two
// buffer modes for input tensors of 2 GiB and more.
// IG_TAP_*: the buffer gather for tap-major layers (see igemm_pack_filter_kernel).
enum { IG_GATHER = 0, IG_POINTWISE = 1, IG_BUF_MASKED = 2, IG_TAP_MASKED = 3, IG_TAP_INSIDE = 4 };

// PW: pointwise layers (1x1, stride 1, no padding: the column matrix IS the input, row c of it
// is channel c of x, contiguous over the pixels) whose pixels-per-image count is a multiple of 4
// and whose channel count is a multiple of BK copy the B tile as 16-byte vectors, unconditionally:
// a pixel group past the end re-reads the last group (its columns are never stored).
template <class TL, int MODE>
__global__ __launch_bounds__(TL::THREADS, TL::MIN_WAVES) void igemm_conv_kernel(const IgemmParams p) {
    constexpr bool PW = MODE == IG_POINTWISE, TAP = MODE == IG_TAP_MASKED || MODE == IG_TAP_INSIDE;
    constexpr bool BUF = MODE == IG_BUF_MASKED || TAP;
    constexpr int BM = TL::BM_, BN = TL::BN_, BK = TL::BK_;
    constexpr int MI = TL::MI, NI = TL::NI, A_LD = TL::A_LD, B_LD = TL::B_LD;
    __shared__ __attribute__((aligned(16))) float As[2][BK * BM];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * BN];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm0 = (wave / TL::WGN_) * TL::WM, wn0 = (wave % TL::WGN_) * TL::WN;
    // Workgroups are dealt to the 8 XCDs round-robin by linear id, and every XCD has an L2 of its own.
    // Tiles are numbered pixel block major, output-channel block minor, and every XCD owns a contiguous
    // eighth of that sequence: the output-channel blocks that share one block of gathered pixels run
    // side by side on ONE XCD and find the pixels in its L2 (dealt round-robin, every XCD would fetch
    // every pixel block: measured 4-6x the algorithmic traffic on the ResNet-50 projections).
    const int nTiles = p.nKB * p.nPB, perXcd = (nTiles + 7) >> 3;
    const int tileId = (blockIdx.x & 7) * perXcd + (blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= perXcd || tileId >= nTiles) return;
    const int pb = tileId / p.nKB, kb = tileId - pb * p.nKB;

    // filter tile: straight 16-byte copies
    const int arow = tid / (BM / 4), acol = (tid % (BM / 4)) * 4;
    const float *ag = p.Wp + (size_t)kb * BM;                     // uniform; the lane adds aOff bytes
    const uint32_t aOff = 4u * ((uint32_t)arow * (uint32_t)p.K_pad + acol);
    const size_t aStage = (size_t)BK * p.K_pad, aPass = (size_t)TL::A_ROWS * p.K_pad;
    const int aLds = arow * BM + acol;

    // the pixel column this thread gathers; its wavefront shares the row
    const int gcol = tid % BN;
    const int grow0 = __builtin_amdgcn_readfirstlane(tid / BN);
    const long pix = (long)pb * BN + gcol;
    const float *ximg = p.x;
    int pixOff = 0;
    uint32_t maskR = 0, maskS = 0;
    if (pix < p.Npix) {
        const uint32_t n = fc_div((uint32_t)pix, p.divOHW);
        const uint32_t pp = (uint32_t)pix - n * (uint32_t)(p.OH * p.OW);
        const uint32_t oh = fc_div(pp, p.divOW), ow = pp - oh * p.OW;
        const int ih0 = (int)oh * p.sh - p.pt, iw0 = (int)ow * p.sw - p.pl;
        ximg = p.x + (size_t)n * p.C * p.H * p.W;
        pixOff = ih0 * p.W + iw0;
        // bit r of maskR: row ih0 + r is inside the image (likewise maskS for columns)
        for (int r = 0; r < p.kh; r++) maskR |= ((unsigned)(ih0 + r) < (unsigned)p.H) ? (1u << r) : 0u;
        for (int q = 0; q < p.kw; q++) maskS |= ((unsigned)(iw0 + q) < (unsigned)p.W) ? (1u << q) : 0u;
    }
    // buffer modes: byte offset of the window origin in the whole tensor, and the taps outside the image
    uint32_t pixByte = 0, invLo = ~0u, invHi = ~0u;
    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.x), 0, BUF ? (int)p.xBytes : 0, 0x00020000);
    if (BUF && pix < p.Npix) {
        pixByte = 4u * (uint32_t)((long)(ximg - p.x) + pixOff);
        if (MODE == IG_BUF_MASKED || MODE == IG_TAP_MASKED) {
            const uint32_t rowBits = ~maskS & ((1u << p.kw) - 1u);      // taps of one window row outside the image
            uint64_t inv = 0;
            for (int r = 0; r < p.kh; r++) {
                const uint32_t bits = ((maskR >> r) & 1u) ? rowBits : ((1u << p.kw) - 1u);
                if (r * p.kw < 64) inv |= (uint64_t)bits << (r * p.kw);
            }
            if (p.kh * p.kw < 64) inv |= ~0ull << (p.kh * p.kw);
            invLo = (uint32_t)inv;
            invHi = (uint32_t)(inv >> 32);
        }
    }
    const int bLds = grow0 * BN + gcol;

    // pointwise: this thread's 4-pixel column group and first row of each copy pass
    constexpr int BV_LD = BK * BN / 4 / TL::THREADS, BV_ROWS = TL::THREADS * 4 / BN;
    static_assert((BK * BN / 4) % TL::THREADS == 0, "every thread copies the same number of float4");
    using SeqBV = std::make_integer_sequence<int, BV_LD>;
    const int vrow = tid / (BN / 4), vcol = (tid % (BN / 4)) * 4;
    const int HW = p.H * p.W;
    const float *vg = p.x;      // uniform; the lane adds vOff bytes (the pointwise path is taken for inputs below 4 GiB)
    uint32_t vOff = 0;
    if (PW) {
        const long pix4 = min((long)pb * BN + vcol, p.Npix - 4);
        const uint32_t n = fc_div((uint32_t)pix4, p.divOHW);
        vOff = 4u * ((n * (uint32_t)p.C + vrow) * (uint32_t)HW + ((uint32_t)pix4 - n * (uint32_t)HW));
    }
    const size_t vPass = (size_t)BV_ROWS * HW, vStage = (size_t)BK * HW;
    const int vLds = vrow * BN + vcol;
    floatx4 rv[BV_LD];

    using SeqA = std::make_integer_sequence<int, A_LD>;
    using SeqB = std::make_integer_sequence<int, B_LD>;
    floatx4 ra[A_LD];
    float rb[B_LD];
    uint32_t rbOk = 0;      // bit i: rb[i] lies inside the image
    // this block's share of the reduction
    const int nStagesAll = p.Kred_pad / BK;
    const int sBegin = blockIdx.y * p.stagesPerSplit, sEnd = min(sBegin + p.stagesPerSplit, nStagesAll);
    // Tap-major gather: the BK rows of a stage are channels tapC .. tapC+BK-1 of one tap (tapR, tapS).
    // Stages are gathered in order, so the tap and the channel are running counters, wave-uniform
    // (scalar registers); only the last addition of an element's offset is per lane.
    const uint32_t chanStep = 4u * (uint32_t)(p.H * p.W);
    int tapT = 0, tapR = 0, tapS = 0, tapC = 0;
    if (TAP) {
        const int stagesPerTap = p.C / BK;          // tap-major layers only: C % BK == 0
        tapT = sBegin / stagesPerTap;
        tapC = (sBegin - tapT * stagesPerTap) * BK;
        tapR = tapT / p.kw;
        tapS = tapT - tapR * p.kw;
    }
    auto tap_gather = [&]() __attribute__((always_inline)) {
        const uint32_t voff = pixByte + 4u * (uint32_t)(tapR * p.W + tapS);
        // the poison bit goes on last: the window origin of a border pixel is a negative (wrapped) offset,
        // and adding a channel to an already poisoned offset could carry out of bit 31 again
        uint32_t poison = 0;
        if (MODE == IG_TAP_MASKED) {
            const uint32_t word = tapT < 32 ? invLo : invHi;
            poison = ((word >> (tapT & 31)) & 1u) << 31;
        }
        const uint32_t chan0 = (uint32_t)(tapC + grow0) * chanStep;
#pragma unroll
        for (int i = 0; i < B_LD; i++)
            rb[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                        xres, (voff + (chan0 + (uint32_t)(i * TL::ROW_STEP) * chanStep)) | poison, 0, 0));
        tapC += BK;
        if (tapC == p.C) {
            tapC = 0;
            tapT++;
            if (++tapS == p.kw) { tapS = 0; tapR++; }
        }
    };
    ag += (size_t)sBegin * aStage;
    ig_load_rows_at(ra, ag, aOff, aPass, SeqA());
    if (PW) {
        vg += (size_t)sBegin * vStage;
        ig_load_rows_at(rv, vg, vOff, vPass, SeqBV());
    } else if (TAP) {
        tap_gather();
    } else if (BUF) {
        ig_gather_rows_buf<true>(rb, xres, pixByte, invLo, invHi, p.table, sBegin * BK + grow0, TL::ROW_STEP, p.kw, SeqB());
    } else {
        rbOk = ig_gather_rows<true>(rb, ximg, pixOff, maskR, maskS, p.table, sBegin * BK + grow0, TL::ROW_STEP, SeqB());
    }

    floatx16 acc[MI][NI];
#pragma unroll
    for (int mi = 0; mi < MI; mi++)
#pragma unroll
        for (int ni = 0; ni < NI; ni++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc[mi][ni][i] = 0.f;

    ig_store_rows(&As[0][aLds], ra, TL::A_ROWS * BM, SeqA());
    if (PW) ig_store_rows(&Bs[0][vLds], rv, BV_ROWS * BN, SeqBV());
    else ig_scatter_rows<!BUF>(&Bs[0][bLds], rb, rbOk, TL::ROW_STEP * BN, SeqB());
    // stage s of the reduction into the staging registers (stages are requested in order: the operands' bases are
    // running pointers in scalar registers, one stage further per call)
    const float *agNext = uniform_ptr(ag + aStage), *vgNext = uniform_ptr(vg + vStage);
    auto load_stage = [&](const int s) __attribute__((always_inline)) {
        ig_load_rows_at(ra, agNext, aOff, aPass, SeqA());
        agNext = uniform_ptr(agNext + aStage);
        if (PW) {
            ig_load_rows_at(rv, vgNext, vOff, vPass, SeqBV());
            vgNext = uniform_ptr(vgNext + vStage);
        }
        else if (TAP) tap_gather();
        else if (BUF) ig_gather_rows_buf<true>(rb, xres, pixByte, invLo, invHi, p.table, s * BK + grow0, TL::ROW_STEP, p.kw, SeqB());
        else rbOk = ig_gather_rows<true>(rb, ximg, pixOff, maskR, maskS, p.table, s * BK + grow0, TL::ROW_STEP, SeqB());
    };
    if (sBegin + 1 < sEnd) load_stage(sBegin + 1);
    __syncthreads();

    const int lrow = lane >> 5, lcol = lane & 31;
    const int aFrag = lrow * BM + wm0 + lcol, bFrag = lrow * BN + wn0 + lcol;
    for (int s = sBegin; s < sEnd; s++) {
        const int buf = (s - sBegin) & 1;
        const float *as = As[buf], *bs = Bs[buf];
        const bool more = s + 1 < sEnd;
        // fragments two reduction steps (kk, kk+2) at a time, a pair ahead of their MFMAs: one ds_read2st64 per
        // 32-wide block and pair, both offsets immediates off an opaque base register (see wino_gemm.hip)
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
            // the reads of the next pair are issued before the MFMAs of this one
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
                // and the one after it is requested at once: a whole stage in flight
                ig_store_rows(&As[buf ^ 1][aLds], ra, TL::A_ROWS * BM, SeqA());
                if (PW) ig_store_rows(&Bs[buf ^ 1][vLds], rv, BV_ROWS * BN, SeqBV());
                else ig_scatter_rows<!BUF>(&Bs[buf ^ 1][bLds], rb, rbOk, TL::ROW_STEP * BN, SeqB());
                if (s + 2 < sEnd) load_stage(s + 2);
            }
        }
        __syncthreads();
    }

    // epilogue: column = pixel (lane%32), rows = output channels.  Register i of an accumulator
    // block is row 8*(i/4) + 4*(lane/32) + i%4: element (row r, column c) of the tile goes to
    // dst[colOff(c) + (rowBase + r) * rowStride], with dst = y (colOff = n*K*OHW + pixel in image,
    // rowStride = OHW) or the partial-sum slab of this split (colOff = pixel, rowStride = Npix).
    const int OHW = p.OH * p.OW;
    const bool partial = p.splitK > 1;
    const int rowBase = kb * BM + wm0 + 4 * lrow;
    if (p.fastStore) {
        // every row of the tile is a real output channel and every byte offset fits 32 bits: a
        // scalar base, one 32-bit offset per store, no predicates
        char *dst = reinterpret_cast<char *>(partial ? p.ws : p.y);
        const uint32_t rowStride = 4u * (partial ? (uint32_t)p.Npix : (uint32_t)OHW);      // bytes
        const uint32_t slab = partial ? (uint32_t)blockIdx.y * (uint32_t)p.K * (uint32_t)p.Npix : 0u;
        const bool plain = partial || (p.bias == nullptr && !p.relu);
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            const long opix = (long)pb * BN + wn0 + ni * 32 + lcol;
            if (opix >= p.Npix) continue;
            uint32_t off;
            if (partial) {
                off = slab + (uint32_t)opix;
            } else {
                const uint32_t n = fc_div((uint32_t)opix, p.divOHW);
                off = n * (uint32_t)p.K * (uint32_t)OHW + ((uint32_t)opix - n * (uint32_t)OHW);
            }
            off = 4u * off + (uint32_t)rowBase * rowStride;
            if (plain) {
#pragma unroll
                for (int mi = 0; mi < MI; mi++)
#pragma unroll
                    for (int i = 0; i < 16; i++)
                        *reinterpret_cast<float *>(dst + (off + (uint32_t)(mi * 32 + 8 * (i / 4) + (i % 4)) * rowStride)) = acc[mi][ni][i];
            } else {
#pragma unroll
                for (int mi = 0; mi < MI; mi++)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        floatx4 bq = {0.f, 0.f, 0.f, 0.f};
                        if (p.bias) bq = *reinterpret_cast<const floatx4 *>(p.bias + rowBase + mi * 32 + 8 * q);
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            float v = acc[mi][ni][q * 4 + j] + bq[j];
                            if (p.relu) v = __builtin_elementwise_maximum(v, 0.f);      // keeps a NaN
                            *reinterpret_cast<float *>(dst + (off + (uint32_t)(mi * 32 + 8 * q + j) * rowStride)) = v;
                        }
                    }
            }
        }
        return;
    }
    if (partial) {
        // partial sums, [split][k][pixel]; igemm_reduce_kernel adds them up in split order
        float *wz = p.ws + (size_t)blockIdx.y * p.K * p.Npix;
#pragma unroll
        for (int ni = 0; ni < NI; ni++) {
            const long opix = (long)pb * BN + wn0 + ni * 32 + lcol;
            if (opix >= p.Npix) continue;
#pragma unroll
            for (int mi = 0; mi < MI; mi++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int k = rowBase + mi * 32 + 8 * (i / 4) + (i % 4);
                    if (k < p.K) wz[(size_t)k * p.Npix + opix] = acc[mi][ni][i];
                }
        }
        return;
    }
#pragma unroll
    for (int ni = 0; ni < NI; ni++) {
        const long opix = (long)pb * BN + wn0 + ni * 32 + lcol;
        if (opix >= p.Npix) continue;
        const uint32_t n = fc_div((uint32_t)opix, p.divOHW);
        const uint32_t pp = (uint32_t)opix - n * (uint32_t)OHW;
        float *yn = p.y + (size_t)n * p.K * OHW + pp;
#pragma unroll
        for (int mi = 0; mi < MI; mi++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int k = rowBase + mi * 32 + 8 * (i / 4) + (i % 4);
                if (k < p.K) {
                    float v = acc[mi][ni][i];
                    if (p.bias) v += p.bias[k];
                    if (p.relu) v = __builtin_elementwise_maximum(v, 0.f);      // keeps a NaN
                    yn[(size_t)k * OHW] = v;
                }
            }
    }
}

// Sums the partial results of a split reduction in split order (so the result does
// not depend on which workgroup finished first), adds bias, applies ReLU, writes NCHW.
__global__ __launch_bounds__(256) void igemm_reduce_kernel(const float *__restrict__ ws, const float *__restrict__ bias,
                                                           float *__restrict__ y, int K, long Npix, int OHW,
                                                           int splitK, int relu, fc_fastdiv divOHW) {
    const long pix = (long)blockIdx.x * 256 + threadIdx.x;
    const int k = blockIdx.y;
    if (pix >= Npix) return;
    const size_t slab = (size_t)K * Npix;
    const float *src = ws + (size_t)k * Npix + pix;
    float v = src[0];
    for (int z = 1; z < splitK; z++) v += src[(size_t)z * slab];
    if (bias) v += bias[k];
    if (relu) v = __builtin_elementwise_maximum(v, 0.f);      // keeps a NaN
    const uint32_t n = fc_div((uint32_t)pix, divOHW);
    y[((size_t)n * K + k) * OHW + (pix - (long)n * OHW)] = v;
}

typedef IgTile<128, 128, 16, 2, 2> Ig0;
typedef IgTile<64, 128, 16, 1, 2> Ig1;
typedef IgTile<128, 64, 16, 2, 1> Ig2;
typedef IgTile<64, 64, 16, 2, 2> Ig3;
typedef IgTile<32, 64, 16, 1, 1> Ig4;
typedef IgTile<256, 128, 16, 2, 2> Ig5;
typedef IgTile<128, 256, 16, 2, 2> Ig6;
typedef IgTile<64, 256, 16, 1, 4> Ig7;

const fc_gemm_config kIgConfigs[] = {
#define FC_CFG(id, T) {id, T::BM_, T::BN_, T::BK_, T::WGM_, T::WGN_, T::LDS_BYTES, 1}
    FC_CFG(0, Ig0), FC_CFG(1, Ig1), FC_CFG(2, Ig2), FC_CFG(3, Ig3),
    FC_CFG(4, Ig4), FC_CFG(5, Ig5), FC_CFG(6, Ig6), FC_CFG(7, Ig7),
#undef FC_CFG
};
const int kNumIgConfigs = sizeof(kIgConfigs) / sizeof(kIgConfigs[0]);

template <class TL>
void launch(fc_context *ctx, IgemmParams &p) {
    const dim3 grid((unsigned)(((p.nKB * p.nPB + 7) / 8) * 8), (unsigned)p.splitK);
    const bool pointwise = p.kh == 1 && p.kw == 1 && p.sh == 1 && p.sw == 1 && p.pt == 0 && p.pl == 0 &&
                           p.OH == p.H && p.OW == p.W && (p.H * p.W) % 4 == 0 && p.C % TL::BK_ == 0 &&
                           ((uintptr_t)p.x & 15) == 0 && p.xBytes < (1l << 32);
    // no tap of any window leaves the image, and no padding rows in the reduction
    const bool inside = p.pt == 0 && p.pl == 0 && (p.OH - 1) * p.sh + p.kh <= p.H && (p.OW - 1) * p.sw + p.kw <= p.W &&
                        (p.C * p.kh * p.kw) % TL::BK_ == 0;
    // one 32-bit byte offset with bit 31 to spare reaches every element of the tensor
    const bool buffer = p.xBytes < (1l << 31);
    const bool tapMajor = p.C % TL::BK_ == 0;      // the order fc_igemm_pack_filter laid the filter out in
    if (pointwise) igemm_conv_kernel<TL, IG_POINTWISE><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(p);
    else if (buffer && tapMajor && inside) igemm_conv_kernel<TL, IG_TAP_INSIDE><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(p);
    else if (buffer && tapMajor && p.kh * p.kw <= 64) igemm_conv_kernel<TL, IG_TAP_MASKED><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(p);
    else if (buffer && p.kh * p.kw <= 64) igemm_conv_kernel<TL, IG_BUF_MASKED><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(p);      // the taps of a window are one 64-bit mask
    else igemm_conv_kernel<TL, IG_GATHER><<<grid, dim3(TL::THREADS), 0, ctx->stream>>>(p);
}

}  // namespace

// Configuration ids: the LDS-tiled shapes of this file first, then the shapes of implicit_gemm_wavesplit.hip.
extern "C" int fc_igemm_num_configs(void) { return kNumIgConfigs + fc_igemm_ws_num_shapes(); }

extern "C" int fc_igemm_get_config(int id, fc_gemm_config *cfg) {
    if (!cfg || id < 0 || id >= fc_igemm_num_configs()) return FC_ERR_INVALID;
    if (id < kNumIgConfigs) *cfg = kIgConfigs[id];
    else fc_igemm_ws_get_config(id - kNumIgConfigs, id, cfg);
    return FC_OK;
}

// Untuned choice: padded multiply-adds divided by the rate each tile shape sustains relative to
// 64x64x16 (measured on MI355X over pointwise, strided and 3x3 layers at batch 32; the shapes with
// 128 accumulators per wavefront run one or two workgroups per CU and fall far behind) and by how
// evenly the grid fills the chip.
extern "C" int fc_igemm_default_config(const fc_conv_shape *s) {
    if (!fc_shape_ok(s)) return FC_ERR_INVALID;
    static const double kRate[] = {0.93, 0.81, 0.82, 1.00, 0.75, 0.60, 0.62, 0.84};
    static_assert(sizeof(kRate) / sizeof(kRate[0]) == sizeof(kIgConfigs) / sizeof(kIgConfigs[0]), "one rate per configuration");
    const double M = s->K, Kr = (double)s->C * s->kh * s->kw;
    const double Np = (double)s->N * fc_out_dim(s->H, s->pt, s->pb, s->kh, s->sh) * fc_out_dim(s->W, s->pl, s->pr, s->kw, s->sw);
    int best = 0;
    double bestCost = 1e300;
    for (int id = 0; id < kNumIgConfigs; id++) {
        const fc_gemm_config &c = kIgConfigs[id];
        const double mp = ceil(M / c.bm) * c.bm, np = ceil(Np / c.bn) * c.bn, kp = ceil(Kr / c.bk) * c.bk;
        const double blocks = (mp / c.bm) * (np / c.bn);
        const double slots = 256.0 * (c.bm * c.bn > 128 * 128 ? 1 : 4);
        // small layers split their reduction until about 768 workgroups exist (fc_igemm_make_plan)
        const double eff_blocks = blocks < 512 ? 768.0 : blocks;
        const double fill = eff_blocks / (ceil(eff_blocks / slots) * slots);
        const double cost = mp * np * kp / (kRate[id] * (0.8 + 0.2 * fill));
        if (cost < bestCost) { bestCost = cost; best = id; }
    }
    // A layer that this tile shape can only fill the chip with by splitting the reduction over workgroups
    // (a pass of partial sums through memory and a second launch) goes to the kernels that split it inside
    // the workgroup instead, while it is small enough for them.
    fc_igemm_plan plan;
    if (fc_igemm_make_plan(s, best, &plan) == FC_OK && plan.split_k > 1) {
        const int ws = fc_igemm_ws_choose(s, plan.Npix);
        if (ws >= 0) return kNumIgConfigs + ws;
    }
    return best;
}

extern "C" int fc_igemm_make_plan(const fc_conv_shape *s, int config, fc_igemm_plan *plan) {
    if (!plan || !fc_shape_ok(s)) return FC_ERR_INVALID;
    fc_gemm_config cfg;
    const int rc = fc_igemm_get_config(config, &cfg);
    if (rc) return rc;
    if (s->kh > 31 || s->kw > 31) return FC_ERR_UNSUPPORTED;      // the in-image test is a 32-bit mask per axis
    plan->shape = *s;
    plan->OH = fc_out_dim(s->H, s->pt, s->pb, s->kh, s->sh);
    plan->OW = fc_out_dim(s->W, s->pl, s->pr, s->kw, s->sw);
    const long kred = (long)s->C * s->kh * s->kw;
    const long npix = (long)s->N * plan->OH * plan->OW;
    if (kred >= (1l << 28) || npix >= (1l << 31) || (long)s->C * s->H * s->W >= (1l << 31)) return FC_ERR_UNSUPPORTED;
    plan->Kred = (int)kred;
    plan->Kred_pad = (int)fc_round_up(kred, cfg.bk);
    plan->K_pad = (int)fc_round_up(s->K, cfg.bm);
    plan->Npix = npix;
    plan->config = config;
    plan->Wp_bytes = sizeof(float) * (size_t)plan->Kred_pad * plan->K_pad;
    plan->table_bytes = sizeof(int32_t) * 2 * (size_t)plan->Kred_pad;
    if (config >= kNumIgConfigs) {
        // the reduction is split inside the workgroups: one launch, no workspace
        if (!fc_igemm_ws_supports(s)) return FC_ERR_UNSUPPORTED;
        plan->split_k = 1;
        plan->ws_bytes = 0;
        return FC_OK;
    }
    // Small layers do not fill 256 CUs with (K_pad/BM) x (Npix/BN) workgroups: split the
    // reduction until about three workgroups per CU exist, keeping >= 4 LDS stages per part.
    const long blocks = (long)(plan->K_pad / cfg.bm) * ((npix + cfg.bn - 1) / cfg.bn);
    const int stages = plan->Kred_pad / cfg.bk;
    int split = 1;
    // A grid of two to four workgroups per CU is placed unevenly by the dispatcher (some CUs get
    // one more than their share and set the time of the launch): with a long reduction, splitting
    // it to about six per CU is worth the second pass (measured: 3x3 stride-2 layers of ResNet-50
    // at batch 32 -9 %, 2048 -> 512 at 7x7 -6 %; with a short reduction the second pass costs more).
    const bool longReduction = stages >= 64;
    const long below = longReduction ? 1024 : 512, target = longReduction ? 1536 : 768;
    if (blocks < below) {
        split = (int)((target + blocks - 1) / blocks);
        if (split > stages / 4) split = stages / 4;
        if (split > 32) split = 32;
        if (split < 1) split = 1;
    }
    const int per = (stages + split - 1) / split;
    plan->split_k = (stages + per - 1) / per;          // no empty parts
    plan->ws_bytes = plan->split_k > 1 ? sizeof(float) * (size_t)plan->split_k * s->K * npix : 0;
    return FC_OK;
}

static int ig_plan_check(fc_context *ctx, const fc_igemm_plan *plan) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan) return fc_set_error(ctx, FC_ERR_INVALID, "null plan", hipSuccess);
    fc_igemm_plan chk;
    const int rc = fc_igemm_make_plan(&plan->shape, plan->config, &chk);
    if (rc) return fc_set_error(ctx, rc, "plan does not describe a supported layer", hipSuccess);
    if (!fc_same_igemm_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "plan fields were modified after fc_igemm_make_plan", hipSuccess);
    return FC_OK;
}

extern "C" int fc_igemm_pack_filter(fc_context *ctx, const fc_igemm_plan *plan, const float *w_dev, float *Wp_dev,
                                    int32_t *table_dev) {
    const int rc = ig_plan_check(ctx, plan);
    if (rc) return rc;
    if (!w_dev || !Wp_dev || !table_dev) return fc_set_error(ctx, FC_ERR_INVALID, "fc_igemm_pack_filter: null buffer", hipSuccess);
    const fc_conv_shape &s = plan->shape;
    const dim3 grid((plan->K_pad + 63) / 64, (plan->Kred_pad + 3) / 4);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_igemm_pack_filter: reduction too long", hipSuccess);
    if (plan->config >= kNumIgConfigs) return fc_igemm_ws_pack(ctx, plan, w_dev, Wp_dev, table_dev);
    fc_gemm_config cfg;
    fc_igemm_get_config(plan->config, &cfg);
    const int tapMajor = s.C % cfg.bk == 0 ? 1 : 0;      // must match the kernel's choice in launch()
    fc_stage_scope scope(ctx, FC_STAGE_FILTER_PACK);
    igemm_pack_filter_kernel<<<grid, dim3(256), 0, ctx->stream>>>(w_dev, Wp_dev, table_dev, s.K, s.C, s.kh, s.kw, s.H,
                                                                 s.W, plan->Kred, plan->Kred_pad, plan->K_pad, tapMajor);
    FC_LAUNCH_CHECK(ctx, "igemm_pack_filter_kernel");
    return FC_OK;
}

// Launches of one layer; `timed` brackets the GEMM kernel with events when stage timing is on.
static int igemm_run(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev, const float *Wp_dev,
                     const int32_t *table_dev, const float *bias_dev, int relu, float *ws_dev, float *y_dev, bool timed,
                     const char *entry);

extern "C" int fc_conv_implicit_gemm(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev,
                                     const float *Wp_dev, const int32_t *table_dev, const float *bias_dev, int relu,
                                     float *ws_dev, float *y_dev) {
    const int rc = ig_plan_check(ctx, plan);
    if (rc) return rc;
    return igemm_run(ctx, plan, x_dev, Wp_dev, table_dev, bias_dev, relu, ws_dev, y_dev, true, "fc_conv_implicit_gemm");
}

// ---- the same layer with the split-reduction workspace in a static device array ----

// Partial sums of a split reduction, [split][K][N*OH*OW] floats, for callers that cannot allocate.
// Every GPU the library runs on holds its own copy of this array until the process ends.
static __device__ __align__(256) float scratch[FC_IGEMM_STATIC_WS_BYTES / sizeof(float)];

// Device address of `scratch` per device, looked up once per device with that device current.
static const int kMaxDevices = 64;
static float *g_scratch_ptr[kMaxDevices];
static bool g_scratch_known[kMaxDevices];
// The context that uses the array of a device: the first one to call fc_conv_implicit_gemm_static there, until it is
// destroyed.  Calls of one context are ordered on its stream; another context's would race with them, so they are refused.
static fc_context *g_scratch_owner[kMaxDevices];
static std::mutex g_scratch_mutex;

// Called by fc_destroy.
void fc_igemm_static_release(fc_context *ctx) {
    if (ctx->device < 0 || ctx->device >= kMaxDevices) return;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_owner[ctx->device] == ctx) g_scratch_owner[ctx->device] = nullptr;
}

// Called by fc_init with ctx->device current.
int fc_igemm_static_init(fc_context *ctx) {
    if (ctx->device < 0 || ctx->device >= kMaxDevices)
        return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_igemm_static_init: device index above 63", hipSuccess);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_known[ctx->device]) {
        float *ptr = nullptr;
        FC_HIP_CHECK(ctx, hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fc_set_error(ctx, FC_ERR_HIP, "fc_igemm_static_init: null address of the static workspace", hipSuccess);
        g_scratch_ptr[ctx->device] = ptr;
        g_scratch_known[ctx->device] = true;
    }
    ctx->igemm_static_ws = g_scratch_ptr[ctx->device];
    return FC_OK;
}

extern "C" int fc_conv_implicit_gemm_static(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev,
                                            const float *Wp_dev, const int32_t *table_dev, const float *bias_dev,
                                            int relu, float *y_dev) {
    const int rc = ig_plan_check(ctx, plan);
    if (rc) return rc;
    if (plan->ws_bytes > (size_t)FC_IGEMM_STATIC_WS_BYTES) {
        char msg[200];
        snprintf(msg, sizeof msg, "fc_conv_implicit_gemm_static: this layer needs %zu bytes of split-reduction workspace, "
                 "the static one holds %d: use fc_conv_implicit_gemm with a workspace of the caller's", plan->ws_bytes,
                 FC_IGEMM_STATIC_WS_BYTES);
        return fc_set_error(ctx, FC_ERR_UNSUPPORTED, msg, hipSuccess);
    }
    if (!ctx->igemm_static_ws) return fc_set_error(ctx, FC_ERR_STATE, "fc_conv_implicit_gemm_static: static workspace not set up", hipSuccess);
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        fc_context *&owner = g_scratch_owner[ctx->device];
        if (owner == nullptr) owner = ctx;
        if (owner != ctx)
            return fc_set_error(ctx, FC_ERR_STATE, "fc_conv_implicit_gemm_static: the static workspace of this GPU is in use by another "
                                "context (one context per GPU may use it at a time; it is free again once that context is destroyed)", hipSuccess);
    }
    // Nothing has to start at zero: every partial sum the reduction reads ([split][k < K][pixel < Npix]) is
    // written by this call's GEMM kernel first.  No event brackets (creating an event may allocate).
    return igemm_run(ctx, plan, x_dev, Wp_dev, table_dev, bias_dev, relu, ctx->igemm_static_ws, y_dev, false,
                     "fc_conv_implicit_gemm_static");
}

static int igemm_run(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev, const float *Wp_dev,
                     const int32_t *table_dev, const float *bias_dev, int relu, float *ws_dev, float *y_dev, bool timed,
                     const char *entry) {
    char msg[160];
    auto fail = [&](int status, const char *what) {
        snprintf(msg, sizeof msg, "%s: %s", entry, what);
        return fc_set_error(ctx, status, msg, hipSuccess);
    };
    if (!x_dev || !Wp_dev || !table_dev || !y_dev) return fail(FC_ERR_INVALID, "null buffer");
    if ((uintptr_t)Wp_dev & 15) return fail(FC_ERR_INVALID, "Wp must be 16-byte aligned");
    if (plan->split_k > 1 && !ws_dev) return fail(FC_ERR_INVALID, "this plan splits the reduction and needs ws_bytes of workspace");
    if (plan->config >= kNumIgConfigs)
        return fc_igemm_ws_run(ctx, plan, plan->config - kNumIgConfigs, x_dev, Wp_dev, table_dev, bias_dev, relu, y_dev, timed);
    fc_gemm_config cfg;
    fc_igemm_get_config(plan->config, &cfg);
    const fc_conv_shape &s = plan->shape;
    IgemmParams p;
    p.x = x_dev; p.Wp = Wp_dev; p.table = table_dev; p.bias = bias_dev; p.y = y_dev;
    p.N = s.N; p.C = s.C; p.H = s.H; p.W = s.W; p.K = s.K; p.OH = plan->OH; p.OW = plan->OW;
    p.kh = s.kh; p.kw = s.kw; p.sh = s.sh; p.sw = s.sw; p.pt = s.pt; p.pl = s.pl; p.relu = relu;
    p.Kred_pad = plan->Kred_pad; p.K_pad = plan->K_pad; p.Npix = plan->Npix;
    p.xBytes = 4l * s.N * s.C * s.H * s.W;
    p.nKB = plan->K_pad / cfg.bm;
    p.nPB = (int)((plan->Npix + cfg.bn - 1) / cfg.bn);
    p.divOHW = fc_make_fastdiv((uint32_t)(plan->OH * plan->OW));
    p.divOW = fc_make_fastdiv((uint32_t)plan->OW);
    p.splitK = plan->split_k;
    p.stagesPerSplit = ((plan->Kred_pad / cfg.bk) + plan->split_k - 1) / plan->split_k;
    p.ws = ws_dev;
    p.fastStore = s.K % cfg.bm == 0 && 4.0 * s.N * s.K * plan->OH * plan->OW < 4294967296.0 &&
                  4.0 * plan->split_k * s.K * (double)plan->Npix < 4294967296.0 && ((uintptr_t)bias_dev & 15) == 0;
    if ((long)p.nKB * p.nPB >= (1l << 31)) return fail(FC_ERR_UNSUPPORTED, "grid too large");
    fc_stage_scope scope(ctx, timed ? FC_STAGE_IMPLICIT_GEMM : -1);
    switch (plan->config) {
        case 0: launch<Ig0>(ctx, p); break;
        case 1: launch<Ig1>(ctx, p); break;
        case 2: launch<Ig2>(ctx, p); break;
        case 3: launch<Ig3>(ctx, p); break;
        case 4: launch<Ig4>(ctx, p); break;
        case 5: launch<Ig5>(ctx, p); break;
        case 6: launch<Ig6>(ctx, p); break;
        case 7: launch<Ig7>(ctx, p); break;
        default: return fail(FC_ERR_INVALID, "unknown tile configuration");
    }
    FC_LAUNCH_CHECK(ctx, "igemm_conv_kernel");
    if (plan->split_k > 1) {
        const dim3 rgrid((unsigned)((plan->Npix + 255) / 256), (unsigned)s.K);
        if (rgrid.y > 65535) return fail(FC_ERR_UNSUPPORTED, "more than 65535 channels");
        igemm_reduce_kernel<<<rgrid, dim3(256), 0, ctx->stream>>>(ws_dev, bias_dev, y_dev, s.K, plan->Npix,
                                                                  plan->OH * plan->OW, plan->split_k, relu, p.divOHW);
        FC_LAUNCH_CHECK(ctx, "igemm_reduce_kernel");
    }
    return FC_OK;
}
