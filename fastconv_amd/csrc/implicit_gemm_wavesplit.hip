// Implicit-GEMM convolution for layers with few output pixels (batch 1): small output tiles, the
// reduction split over the wavefronts of ONE workgroup.
//
// A layer such as 2048 -> 512 channels at 7x7 has 49 output pixels: under 64x64 tiles it is 8
// workgroups, and filling the chip by splitting the reduction over workgroups costs a pass of
// partial sums through memory and a second launch to add them.  Here a workgroup owns a tile of
// 16*MT output channels x 16*NT pixels (v_mfma_f32_16x16x4_f32 blocks), so that a few hundred
// workgroups exist, and its NW wavefronts take the 16-row units of the reduction in turn (wavefront
// w: units w, w + NW, ...).  Wavefronts share no operand, so nothing is staged in LDS: both operands
// go from L2 straight into the registers the MFMA takes them from, several units ahead.  At the end
// the NW partial tiles meet in LDS and are added in wavefront order (a fixed order: results do not
// depend on timing), bias and ReLU are applied and y is written.  One launch per layer.
//
// Operand layouts (row = output channel, col = pixel, depth = reduction index inside a unit):
//   A, lane l of step j:  filter value of channel 16*block + l % 16, reduction row 16*u + 4*(l / 16) + j.
//      The filter is re-laid once to Wq[K_pad/16][units][64 lanes][4 steps]: one 16-byte load per
//      lane, unit and channel block (1 KB contiguous per wavefront).
//   B, lane l of step j:  input element of pixel l % 16 for the same reduction row, gathered through a
//      buffer resource over x (one 32-bit byte offset; taps outside the image get bit 31 set and the
//      hardware's range check answers 0), as in igemm_conv_kernel.
//   D, lane l, register i: channel 4*(l / 16) + i, pixel l % 16.
#include <cstdio>

#include "fc_internal.h"

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

struct WsParams {
    const float *x;
    const float *Wq;
    const int32_t *table;
    const float *bias;
    float *y;
    int C, H, W, K, OH, OW, kh, kw, sh, sw, pt, pl, relu;
    int nUnits;           // 16-row units of the (padded) reduction
    int nKB, nPB;         // tiles along output channels and pixels
    int pixFastest;       // tile order inside an XCD's range: pixel block fastest (the filter is the larger operand) or channel block fastest
    int unitsPerTap;      // tap-major layers: C / 16
    int xBytes, wqBytes;
    long Npix;
    uint32_t chanStep;    // bytes between channels of x
    fc_fastdiv divOHW, divOW, divUnitsPerTap, divKw;
};

// How the reduction rows of a unit map to elements of x.
//   WS_TAP_*: tap-major order (C a multiple of 16): the 16 rows of a unit are 16 consecutive channels of one
//             filter tap; tap and first channel follow from the unit number in scalar registers.
//   WS_TABLE: any order, through the row table (offset from the window origin, r << 16 | s).
//   WS_ROW3:  tap-major layers with 3 taps per window row: the three taps of a window row are three consecutive
//             floats of x, so one 12-byte load per (channel, pixel, window row) feeds three units -- a third of the
//             gather instructions of WS_TAP_MASKED, and instruction issue is what a workgroup runs out of.
enum { WS_TAP_INSIDE = 0, WS_TAP_MASKED = 1, WS_TABLE = 2, WS_ROW3 = 3 };

template <int MT, int NT, int NW, int MODE>
__global__ __launch_bounds__(64 * NW) void igemm_wavesplit_kernel(const WsParams p) {
    // Units requested ahead per wavefront.  Shallow on purpose: with 8 to 20 wavefronts on a CU the latencies are
    // covered by the other wavefronts, and what a CU runs out of is vector-memory instruction issue (a 64-lane
    // load occupies the address unit for about 16 cycles whatever its width), which deeper prefetch only adds to
    // (measured over the batch-1 ResNet-50 layers: 2/1 units ahead 378 us, 3/2 392, 4/2 399, 6/3 423).
    constexpr int PF = MT * NT >= 4 ? 1 : 2;
    constexpr int TILE = MT * NT * 256;           // floats of one wavefront's partial tile
    __shared__ __attribute__((aligned(16))) float red[NW * TILE];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6);
    const int g = lane >> 4, col = lane & 15;
    // every XCD (workgroups are dealt to them round robin) owns a contiguous range of tiles, numbered
    // so that the tiles sharing the larger operand sit side by side and meet in one L2
    const int nTiles = p.nKB * p.nPB, perXcd = (nTiles + 7) >> 3;
    const int tileId = (int)(blockIdx.x & 7) * perXcd + (int)(blockIdx.x >> 3);
    if ((int)(blockIdx.x >> 3) >= perXcd || tileId >= nTiles) return;
    int kb, pb;
    if (p.pixFastest) {
        kb = tileId / p.nPB;
        pb = tileId - kb * p.nPB;
    } else {
        pb = tileId / p.nKB;
        kb = tileId - pb * p.nKB;
    }

    // this lane's pixel in each of the NT blocks: byte offset of its window origin in x (it may be
    // "negative", i.e. wrapped, for a border pixel) and the taps of the window outside the image
    const int OHW = p.OH * p.OW;
    uint32_t pre[NT], invLo[NT], invHi[NT];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) {
        const long pix = (long)pb * (16 * NT) + nt * 16 + col;
        pre[nt] = 0;
        invLo[nt] = invHi[nt] = ~0u;
        if (pix < p.Npix) {
            const uint32_t n = fc_div((uint32_t)pix, p.divOHW);
            const uint32_t pp = (uint32_t)pix - n * (uint32_t)OHW;
            const uint32_t oh = fc_div(pp, p.divOW), ow = pp - oh * p.OW;
            const int ih0 = (int)oh * p.sh - p.pt, iw0 = (int)ow * p.sw - p.pl;
            pre[nt] = 4u * (n * (uint32_t)(p.C * p.H * p.W) + (uint32_t)(ih0 * p.W + iw0));
            if (MODE != WS_TAP_INSIDE) {
                uint32_t colBits = 0;      // taps of one window row outside the image
                for (int q = 0; q < p.kw; q++) colBits |= ((unsigned)(iw0 + q) < (unsigned)p.W) ? 0u : (1u << q);
                const uint32_t allBits = (1u << p.kw) - 1u;
                uint64_t inv = 0;
                for (int r = 0; r < p.kh; r++) {
                    const uint32_t bits = ((unsigned)(ih0 + r) < (unsigned)p.H) ? colBits : allBits;
                    if (r * p.kw < 64) inv |= (uint64_t)bits << (r * p.kw);
                }
                if (p.kh * p.kw < 64) inv |= ~0ull << (p.kh * p.kw);
                invLo[nt] = (uint32_t)inv;
                invHi[nt] = (uint32_t)(inv >> 32);
            }
        }
        if (MODE != WS_TABLE) pre[nt] += 4u * (uint32_t)g * p.chanStep;      // step j adds j channels
    }
    // WS_ROW3: the load of a window row starts at its first column inside the image (left padding of at most one
    // column: the values then sit one component further left); columns outside the image are zeroed after the load,
    // rows outside poison the whole load.  rowBad: bit r set = window row r outside the image (all set past the last pixel).
    bool shifted[NT], colBad[NT][3];
    uint32_t rowBad[NT];
    if (MODE == WS_ROW3) {
#pragma unroll
        for (int nt = 0; nt < NT; nt++) {
            // bits 0..2 of the tap mask are the columns of window row 0 when that row is inside; rebuilt from the pixel here
            const long pix = (long)pb * (16 * NT) + nt * 16 + col;
            shifted[nt] = false;
            colBad[nt][0] = colBad[nt][1] = colBad[nt][2] = true;
            rowBad[nt] = ~0u;
            if (pix < p.Npix) {
                const uint32_t n = fc_div((uint32_t)pix, p.divOHW);
                const uint32_t pp = (uint32_t)pix - n * (uint32_t)OHW;
                const uint32_t oh = fc_div(pp, p.divOW), ow = pp - oh * p.OW;
                const int ih0 = (int)oh * p.sh - p.pt, iw0 = (int)ow * p.sw - p.pl;
                shifted[nt] = iw0 < 0;
#pragma unroll
                for (int q = 0; q < 3; q++) colBad[nt][q] = !((unsigned)(iw0 + q) < (unsigned)p.W);
                rowBad[nt] = 0;
                for (int r = 0; r < p.kh; r++) rowBad[nt] |= ((unsigned)(ih0 + r) < (unsigned)p.H) ? 0u : (1u << r);
                if (shifted[nt]) pre[nt] += 4u;
            }
        }
    }
    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.x), 0, p.xBytes, 0x00020000);

    __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.Wq), 0, p.wqBytes, 0x00020000);
    const uint32_t aLane = (uint32_t)lane * 16u;
    const uint32_t aBlock = (uint32_t)p.nUnits * 1024u;                 // bytes between channel blocks of Wq
    const uint32_t aTile = (uint32_t)(kb * MT) * aBlock;

    // Requests unit u: MT 16-byte pieces of the filter, 4*NT elements of x.  `dead` is bit 31 for a request past the
    // wavefront's last unit (u is then any valid unit): every offset of it lies outside its buffer, so the loads are
    // issued and return 0 without touching memory.  Loads are never skipped by a branch: where such paths join, the
    // compiler waits for every load in flight.
    auto load = [&](const int u, const uint32_t dead, floatx4 (&a)[MT], float (&b)[NT][4]) __attribute__((always_inline)) {
        const uint32_t aUnit = aTile + (uint32_t)u * 1024u;
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
            a[mt] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wres, (aLane + (aUnit + (uint32_t)mt * aBlock)) | dead, 0, 0));
        if (MODE != WS_TABLE) {
            const uint32_t t = fc_div((uint32_t)u, p.divUnitsPerTap);
            const uint32_t c0 = ((uint32_t)u - t * (uint32_t)p.unitsPerTap) * 16u;
            const uint32_t tr = fc_div(t, p.divKw), ts = t - tr * (uint32_t)p.kw;
            const uint32_t sOff = 4u * (tr * (uint32_t)p.W + ts) + c0 * p.chanStep;
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                // the poison bit goes on last: a border pixel's origin is a wrapped negative offset, and
                // adding to an already poisoned offset could carry out of bit 31 again
                uint32_t poison = dead;
                if (MODE == WS_TAP_MASKED) poison |= (((t < 32u ? invLo[nt] : invHi[nt]) >> (t & 31u)) & 1u) << 31;
#pragma unroll
                for (int j = 0; j < 4; j++)
                    b[nt][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                   xres, (pre[nt] + (sOff + (uint32_t)j * p.chanStep)) | poison, 0, 0));
            }
        } else {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int kr = 16 * u + 4 * g + j;
                const uint32_t off = 4u * (uint32_t)p.table[2 * kr];
                const int rs = p.table[2 * kr + 1];
                const uint32_t t = (uint32_t)(rs >> 16) * (uint32_t)p.kw + (uint32_t)(rs & 0xffff);
#pragma unroll
                for (int nt = 0; nt < NT; nt++) {
                    const uint32_t word = t < 32u ? invLo[nt] : invHi[nt];
                    const uint32_t bad = t < 64u ? (word >> (t & 31u)) & 1u : 1u;
                    b[nt][j] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
                                   xres, (pre[nt] + off) | (bad << 31) | dead, 0, 0));
                }
            }
        }
    };

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++) acc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};

    if (MODE == WS_ROW3) {
        // items of this wavefront: (window row r, block of 16 channels cb) = wave, wave + NW, ...; an item is the three
        // units (r, 0..2) of that channel block
        typedef float floatx3 __attribute__((ext_vector_type(3)));
        const int cpb = p.unitsPerTap, nItems = p.kh * cpb;
        const int myItems = wave < nItems ? (nItems - wave + NW - 1) / NW : 0;
        constexpr int PFR = MT * NT >= 4 ? 1 : 2;
        floatx4 ia[PFR][3][MT];
        floatx3 ib[PFR][NT][4];
        auto requestItem = [&](const int i, floatx4 (&a)[3][MT], floatx3 (&b)[NT][4]) __attribute__((always_inline)) {
            const int it = min(wave + i * NW, nItems - 1);
            const uint32_t dead = i < myItems ? 0u : 0x80000000u;
            const uint32_t r = fc_div((uint32_t)it, p.divUnitsPerTap), cb = (uint32_t)it - r * (uint32_t)cpb;
#pragma unroll
            for (int q = 0; q < 3; q++) {
                const uint32_t aUnit = aTile + ((r * 3u + q) * (uint32_t)cpb + cb) * 1024u;
#pragma unroll
                for (int mt = 0; mt < MT; mt++)
                    a[q][mt] = __builtin_bit_cast(floatx4, __builtin_amdgcn_raw_buffer_load_b128(wres, (aLane + (aUnit + (uint32_t)mt * aBlock)) | dead, 0, 0));
            }
            const uint32_t sOff = 4u * r * (uint32_t)p.W + cb * 16u * p.chanStep;
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                const uint32_t poison = dead | (((rowBad[nt] >> r) & 1u) << 31);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    b[nt][j] = __builtin_bit_cast(floatx3, __builtin_amdgcn_raw_buffer_load_b96(
                                   xres, (pre[nt] + (sOff + (uint32_t)j * p.chanStep)) | poison, 0, 0));
            }
        };
#pragma unroll
        for (int i = 0; i < PFR; i++) requestItem(i, ia[i], ib[i]);
        for (int it = 0; it < myItems; it += PFR) {
#pragma unroll
            for (int i = 0; i < PFR; i++) {
                if (it + i < myItems) {
#pragma unroll
                    for (int nt = 0; nt < NT; nt++)
#pragma unroll
                        for (int j = 0; j < 4; j++) {
                            const floatx3 v = ib[i][nt][j];
                            float t[3];
                            t[0] = colBad[nt][0] ? 0.f : v[0];
                            t[1] = colBad[nt][1] ? 0.f : (shifted[nt] ? v[0] : v[1]);
                            t[2] = colBad[nt][2] ? 0.f : (shifted[nt] ? v[1] : v[2]);
#pragma unroll
                            for (int q = 0; q < 3; q++)
#pragma unroll
                                for (int mt = 0; mt < MT; mt++)
                                    acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ia[i][q][mt][j], t[q], acc[mt][nt], 0, 0, 0);
                        }
                }
                requestItem(it + i + PFR, ia[i], ib[i]);
            }
        }
    } else {
        // units of this wavefront: wave, wave + NW, ...
        const int myUnits = wave < p.nUnits ? (p.nUnits - wave + NW - 1) / NW : 0;
        const int lastUnit = p.nUnits - 1;
        auto request = [&](const int i, floatx4 (&a)[MT], float (&b)[NT][4]) __attribute__((always_inline)) {
            load(min(wave + i * NW, lastUnit), i < myUnits ? 0u : 0x80000000u, a, b);
        };
        floatx4 ra[PF][MT];
        float rb[PF][NT][4];
    #pragma unroll
        for (int i = 0; i < PF; i++) request(i, ra[i], rb[i]);
        for (int it = 0; it < myUnits; it += PF) {
    #pragma unroll
            for (int i = 0; i < PF; i++) {
                if (it + i < myUnits) {
    #pragma unroll
                    for (int j = 0; j < 4; j++)
    #pragma unroll
                        for (int mt = 0; mt < MT; mt++)
    #pragma unroll
                            for (int nt = 0; nt < NT; nt++)
                                acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(ra[i][mt][j], rb[i][nt][j], acc[mt][nt], 0, 0, 0);
                }
                request(it + i + PF, ra[i], rb[i]);
            }
        }
    }

    // the NW partial tiles meet in LDS, [wavefront][block][register][lane], and are added in wavefront order
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
        for (int nt = 0; nt < NT; nt++)
#pragma unroll
            for (int i = 0; i < 4; i++) red[wave * TILE + (mt * NT + nt) * 256 + i * 64 + lane] = acc[mt][nt][i];
    __syncthreads();
    for (int e = threadIdx.x; e < TILE; e += 64 * NW) {
        float v = red[e];
#pragma unroll
        for (int w = 1; w < NW; w++) v += red[w * TILE + e];
        const int blk = e >> 8, i = (e >> 6) & 3, ln = e & 63;
        const int mt = blk / NT, nt = blk - mt * NT;
        const int k = (kb * MT + mt) * 16 + 4 * (ln >> 4) + i;
        const long pix = (long)pb * (16 * NT) + nt * 16 + (ln & 15);
        if (k < p.K && pix < p.Npix) {
            if (p.bias) v += p.bias[k];
            if (p.relu) v = __builtin_elementwise_maximum(v, 0.f);      // keeps a NaN
            const uint32_t n = fc_div((uint32_t)pix, p.divOHW);
            p.y[((size_t)n * p.K + k) * OHW + ((uint32_t)pix - n * (uint32_t)OHW)] = v;
        }
    }
}

// Wq[K_pad/16][units][64][4] and the row table, in the reduction order the layer uses (tap-major when C is
// a multiple of 16, else the column matrix's channel-major order: see igemm_pack_filter_kernel).
__global__ __launch_bounds__(256) void igemm_wavesplit_pack_kernel(const float *__restrict__ w, float *__restrict__ Wq,
                                                                   int32_t *__restrict__ table, int K, int C, int kh, int kw,
                                                                   int H, int W, int Kred, int nUnits, long total, int tapMajor) {
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= total) return;
    const int j = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
    const long bu = idx >> 8;
    const int u = (int)(bu % nUnits), kb16 = (int)(bu / nUnits);
    const int k = kb16 * 16 + (lane & 15), kred = 16 * u + 4 * (lane >> 4) + j;
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
    Wq[idx] = (k < K && kred < Kred) ? w[((size_t)k * C + c) * (kh * kw) + r * kw + s] : 0.f;
    if (kb16 == 0 && (lane & 15) == 0) {
        table[2 * kred] = kred < Kred ? c * H * W + r * W + s : 0;
        table[2 * kred + 1] = (r << 16) | s;
    }
}

struct WsShape {
    int mt, nt, nw;
};
// the configurations after the LDS-tiled ones of implicit_gemm.hip, in the order of their ids
const WsShape kWsShapes[] = {{1, 1, 4}, {1, 1, 8}, {1, 1, 16}, {1, 2, 4}, {1, 2, 8}, {1, 2, 16},
                             {2, 1, 4}, {2, 1, 8}, {2, 1, 16}, {2, 2, 4}, {2, 2, 8}, {2, 2, 16},
                             {4, 2, 4}, {4, 2, 8}, {2, 4, 4}, {2, 4, 8}, {4, 4, 4}};
const int kNumWsShapes = sizeof(kWsShapes) / sizeof(kWsShapes[0]);

template <int MT, int NT, int NW>
void ws_launch(fc_context *ctx, const WsParams &p, int mode) {
    const dim3 grid((unsigned)(((p.nKB * p.nPB + 7) / 8) * 8)), block(64 * NW);
    if (mode == WS_TAP_INSIDE) igemm_wavesplit_kernel<MT, NT, NW, WS_TAP_INSIDE><<<grid, block, 0, ctx->stream>>>(p);
    else if (mode == WS_TAP_MASKED) igemm_wavesplit_kernel<MT, NT, NW, WS_TAP_MASKED><<<grid, block, 0, ctx->stream>>>(p);
    else if (mode == WS_ROW3) igemm_wavesplit_kernel<MT, NT, NW, WS_ROW3><<<grid, block, 0, ctx->stream>>>(p);
    else igemm_wavesplit_kernel<MT, NT, NW, WS_TABLE><<<grid, block, 0, ctx->stream>>>(p);
}

}  // namespace

int fc_igemm_ws_num_shapes() { return kNumWsShapes; }

void fc_igemm_ws_get_config(int index, int id, fc_gemm_config *cfg) {
    const WsShape &s = kWsShapes[index];
    cfg->id = id;
    cfg->bm = 16 * s.mt;
    cfg->bn = 16 * s.nt;
    cfg->bk = 16;
    cfg->waves_m = 1;
    cfg->waves_n = 1;
    cfg->lds_bytes = s.nw * s.mt * s.nt * 1024;
    cfg->waves_k = s.nw;
}

// These kernels gather through a buffer resource with 32-bit offsets (bit 31 to spare) and one 64-bit mask of taps
bool fc_igemm_ws_supports(const fc_conv_shape *s) {
    // (the filter is addressed the same way: K rounded up to 64 at most)
    return 4.0 * s->N * s->C * s->H * s->W < 2147483648.0 && s->kh * s->kw <= 64 &&
           4.0 * (s->K + 63.0) * ((double)s->C * s->kh * s->kw + 15.0) < 2147483648.0;
}

// Untuned choice among these configurations, for a layer whose reduction the LDS-tiled kernels would have to
// split over workgroups; -1 when they should keep the layer.  Read off per-configuration times of the
// ResNet-50 and VGG-16 layers at batch 1 to 32 and of a dozen other shapes on MI355X.  What a workgroup costs
// is vector-memory instruction issue (MT + 4*NT loads per unit whatever their width), so the largest tile
// that still spreads over the chip wins (64x32, 32x32 or 32x16 from 192 workgroups on, else 16x16),
// unless a smaller one pads the layer less.
// 8 wavefronts over the reduction, 4 when it is shorter than 16 units (16 wavefronts are ahead by 3-5 % on a
// few long reductions at batch 8 to 16 and behind by 10 % on 256 -> 256 channels at 56x56: not chosen).  Beyond about 8 GFLOP (2 GFLOP for strided layers, whose
// gathered rows use half of every cache line) the LDS-tiled kernels are level or ahead despite their second launch.
int fc_igemm_ws_choose(const fc_conv_shape *s, long Npix) {
    if (!fc_igemm_ws_supports(s)) return -1;
    const double flops = 2.0 * Npix * s->K * (double)s->C * s->kh * s->kw;
    if (flops > (s->sh > 1 || s->sw > 1 ? 2.0e9 : 8.0e9)) return -1;
    const int nUnits = (s->C * s->kh * s->kw + 15) / 16;
    // among the tiles that bring enough workgroups, the least padded work, weighted by what a product costs in loads
    static const struct { int mt, nt; long minWgs; double weight; } kTiles[4] = {{4, 2, 192, 1.00}, {2, 2, 192, 1.15}, {2, 1, 192, 1.30}, {1, 1, 0, 1.70}};
    int mt = 1, nt = 1;
    double bestCost = 1e300;
    for (int i = 0; i < 4; i++) {
        const long kBlocks = (s->K + 16 * kTiles[i].mt - 1) / (16 * kTiles[i].mt), pBlocks = (Npix + 16 * kTiles[i].nt - 1) / (16 * kTiles[i].nt);
        if (kBlocks * pBlocks < kTiles[i].minWgs) continue;
        const double cost = (double)(kBlocks * 16 * kTiles[i].mt) * (double)(pBlocks * 16 * kTiles[i].nt) * kTiles[i].weight;
        if (cost < bestCost) { bestCost = cost; mt = kTiles[i].mt; nt = kTiles[i].nt; }
    }
    const int nw = nUnits >= 16 ? 8 : 4;
    for (int i = 0; i < kNumWsShapes; i++)
        if (kWsShapes[i].mt == mt && kWsShapes[i].nt == nt && kWsShapes[i].nw == nw) return i;
    return -1;
}

int fc_igemm_ws_pack(fc_context *ctx, const fc_igemm_plan *plan, const float *w_dev, float *Wq_dev, int32_t *table_dev) {
    const fc_conv_shape &s = plan->shape;
    const int nUnits = plan->Kred_pad / 16;
    const long total = (long)(plan->K_pad / 16) * nUnits * 256;
    if ((total + 255) / 256 >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_igemm_pack_filter: filter too large", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_FILTER_PACK);
    igemm_wavesplit_pack_kernel<<<dim3((unsigned)((total + 255) / 256)), dim3(256), 0, ctx->stream>>>(
        w_dev, Wq_dev, table_dev, s.K, s.C, s.kh, s.kw, s.H, s.W, plan->Kred, nUnits, total, s.C % 16 == 0 ? 1 : 0);
    FC_LAUNCH_CHECK(ctx, "igemm_wavesplit_pack_kernel");
    return FC_OK;
}

int fc_igemm_ws_run(fc_context *ctx, const fc_igemm_plan *plan, int index, const float *x_dev, const float *Wq_dev,
                    const int32_t *table_dev, const float *bias_dev, int relu, float *y_dev, bool timed) {
    const fc_conv_shape &s = plan->shape;
    const WsShape &sh = kWsShapes[index];
    WsParams p;
    p.x = x_dev; p.Wq = Wq_dev; p.table = table_dev; p.bias = bias_dev; p.y = y_dev;
    p.C = s.C; p.H = s.H; p.W = s.W; p.K = s.K; p.OH = plan->OH; p.OW = plan->OW;
    p.kh = s.kh; p.kw = s.kw; p.sh = s.sh; p.sw = s.sw; p.pt = s.pt; p.pl = s.pl; p.relu = relu;
    p.nUnits = plan->Kred_pad / 16;
    p.nKB = plan->K_pad / (16 * sh.mt);
    p.nPB = (int)((plan->Npix + 16 * sh.nt - 1) / (16 * sh.nt));
    p.Npix = plan->Npix;
    p.xBytes = (int)(4l * s.N * s.C * s.H * s.W);
    p.wqBytes = (int)plan->Wp_bytes;
    p.chanStep = 4u * (uint32_t)(s.H * s.W);
    const bool tapMajor = s.C % 16 == 0;
    p.unitsPerTap = tapMajor ? s.C / 16 : 1;
    p.divOHW = fc_make_fastdiv((uint32_t)(plan->OH * plan->OW));
    p.divOW = fc_make_fastdiv((uint32_t)plan->OW);
    p.divUnitsPerTap = fc_make_fastdiv((uint32_t)p.unitsPerTap);
    p.divKw = fc_make_fastdiv((uint32_t)s.kw);
    p.pixFastest = (double)plan->Kred_pad * plan->K_pad > (double)s.N * s.C * s.H * s.W ? 1 : 0;
    if ((long)p.nKB * p.nPB >= (1l << 31) - 8) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_conv_implicit_gemm: grid too large", hipSuccess);
    const bool inside = s.pt == 0 && s.pl == 0 && (plan->OH - 1) * s.sh + s.kh <= s.H && (plan->OW - 1) * s.sw + s.kw <= s.W;
    // three taps per window row and at most one column of left padding: a 12-byte load per window row
    const bool row3 = tapMajor && s.kw == 3 && s.pl <= 1 && s.kh <= 31;
    const int mode = !tapMajor ? WS_TABLE : row3 ? WS_ROW3 : inside ? WS_TAP_INSIDE : WS_TAP_MASKED;
    fc_stage_scope scope(ctx, timed ? FC_STAGE_IMPLICIT_GEMM : -1);
#define FC_WS_CASE(I, MT_, NT_, NW_) case I: ws_launch<MT_, NT_, NW_>(ctx, p, mode); break
    switch (index) {
        FC_WS_CASE(0, 1, 1, 4); FC_WS_CASE(1, 1, 1, 8); FC_WS_CASE(2, 1, 1, 16);
        FC_WS_CASE(3, 1, 2, 4); FC_WS_CASE(4, 1, 2, 8); FC_WS_CASE(5, 1, 2, 16);
        FC_WS_CASE(6, 2, 1, 4); FC_WS_CASE(7, 2, 1, 8); FC_WS_CASE(8, 2, 1, 16);
        FC_WS_CASE(9, 2, 2, 4); FC_WS_CASE(10, 2, 2, 8); FC_WS_CASE(11, 2, 2, 16);
        FC_WS_CASE(12, 4, 2, 4); FC_WS_CASE(13, 4, 2, 8); FC_WS_CASE(14, 2, 4, 4); FC_WS_CASE(15, 2, 4, 8); FC_WS_CASE(16, 4, 4, 4);
        default: return fc_set_error(ctx, FC_ERR_INVALID, "fc_conv_implicit_gemm: unknown tile configuration", hipSuccess);
    }
#undef FC_WS_CASE
    FC_LAUNCH_CHECK(ctx, "igemm_wavesplit_kernel");
    return FC_OK;
}
