// Winograd F(6x6,3x3) transform kernels for gfx950: filter (G g G^T), input
// (B^T d B) and output (A^T m A).  All three are HBM-bound; the layouts are
//   U[64][C_pad][K_pad], V[64][C_pad][T_pad], M[64][K_pad][T_pad]
// with the last index fastest, so that a wavefront whose lanes walk consecutive
// output channels (U) or consecutive tiles (V, M) touches 256 contiguous bytes
// per frequency plane.
#include "fc_internal.h"
#include "wino_math.h"

namespace {

// Uniform base pointer + 32-bit byte offset of the lane: the address form that costs no vector
// instruction (the base lives in scalar registers, the offset is one register shared by all the
// loads or stores of the lane).
// M is read exactly once, by the output transform: loaded with the non-temporal hint it does not
// displace what the caches hold for the kernels around it (measured on the batch-32 VGG-16 layers:
// the output transform 6 % shorter over the stack, 14 % on 128 -> 128 channels at 112x112).  The
// same hint on the stores of V makes the input transform 40 % faster when it runs by itself, and
// slower inside the pipeline.
__device__ __forceinline__ float load_m_at(const float *base, uint32_t byteOff) {
    return __builtin_nontemporal_load(reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + byteOff));
}
__device__ __forceinline__ void store_at(float *base, uint32_t byteOff, float v) {
    *reinterpret_cast<float *>(reinterpret_cast<char *>(base) + byteOff) = v;
}

// ---------------------------------------------------------------- filter

// One thread per (output channel, input channel); lanes walk output channels so
// the 64 plane stores of a wavefront are contiguous.
struct FilterTParams {
    const float *w;
    float *U;
    int K, C, K_pad, C_pad;
};

// Block (bx, by) = output channels 64*bx .. +63 of input channels 4*by .. +3.
__device__ __forceinline__ void filter_transform_block(const FilterTParams &q, int bx, int by) {
    const float *__restrict__ w = q.w;
    float *__restrict__ U = q.U;
    const int K = q.K, C = q.C, K_pad = q.K_pad, C_pad = q.C_pad;
    const int lane = threadIdx.x & 63;
    const int k = bx * 64 + lane;
    const int c = by * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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
    float *pf = U + (size_t)c * K_pad + bx * 64;       // uniform; the lane adds 4 * lane
    const uint32_t laneOff = (uint32_t)lane * 4u;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float o[8];
        g8(t[i], o);
#pragma unroll
        for (int j = 0; j < 8; j++) {
            store_at(pf, laneOff, o[j]);
            pf += plane;
        }
    }
}

__global__ __launch_bounds__(256) void wino_filter_transform_kernel(const FilterTParams q) {
    filter_transform_block(q, blockIdx.x, blockIdx.y);
}

// ----------------------------------------------------------------- input

// Tiles are numbered t = (n*tH + th)*tW + tw, so t / tW is a "band": one row of
// tiles of one image, gb = n*tH + th.  Both transform kernels give a workgroup
// TPB consecutive tiles starting at a multiple of TPB, whatever bands and images
// that range crosses: every store to (or load from) a frequency plane is then a
// whole number of aligned 128-byte lines.
struct InTParams {
    const float *x;
    float *V;
    int N, C, H, W, pad_t, pad_l;
    int tH, tW;
    long T;          // real tiles; tiles in [T, T_pad) are written as zeros
    unsigned xBytes; // size of x when it is at most 2 GiB (the buffer path), else unused
    int C_pad;
    long T_pad;
    int LW;          // 6*tW + 2: columns of a band as its tiles see it, padding columns included
    fc_fastdiv divLW, divTH, divTW;
};

// Block = one input channel x TPB consecutive tiles.
// Pass 1 applies B^T down the 8 rows of each band the tile range touches: a
// thread owns up to ITEMS columns (one column of one band each), so the 8 global loads of a wavefront are
// row-contiguous.  Pass 2 applies B along the rows out of LDS: a thread owns one
// tile and 8*TPB/256 of its 8 rows, and stores to the frequency planes with lanes
// on consecutive tiles.
// BUF: x is read through a buffer resource with 32-bit byte offsets; an element outside the image
// (or a column this block does not need) gets an offset with bit 31 set, which is past the end of
// x, and the hardware returns zero: no branch and no 64-bit address per load.  Inputs of more than
// 2 GiB take the pointer path.  The plane stores of pass 2 use a scalar base per frequency and one
// 32-bit lane offset (the kernel spent half of its vector instructions on addresses before).
template <int TPB, int ITEMS, bool BUF>
__device__ __forceinline__ void input_transform_block(const InTParams &p, int bx, int c, float *lds) {
    const int tid = threadIdx.x;
    const size_t plane = (size_t)p.C_pad * p.T_pad;
    const uint32_t t0 = bx * TPB;
    const uint32_t tLast = min((uint32_t)(t0 + TPB), (uint32_t)p.T) - 1;   // last real tile (wraps if none)
    const bool anyReal = t0 < (uint32_t)p.T;
    const uint32_t gb0 = fc_div(t0, p.divTW), gbL = anyReal ? fc_div(tLast, p.divTW) : gb0;
    const int tw0 = t0 - gb0 * p.tW, twL = tLast - gbL * p.tW;
    const int NB = anyReal ? (int)(gbL - gb0) + 1 : 0;

    if (c < p.C) {
        // All global loads of a thread (up to ITEMS columns x 8 rows) are issued before any
        // is consumed: the kernel is latency-bound otherwise (few bytes in flight per CU).
        const int items = NB * p.LW;
        float d[ITEMS][8];
        int dstOff[ITEMS];
        if (BUF) {
            __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.x), 0, (int)p.xBytes, 0x00020000);
            const uint32_t chanOff = (uint32_t)c * (uint32_t)(p.H * p.W);
            const uint32_t imgStride = (uint32_t)p.C * (uint32_t)(p.H * p.W);
#pragma unroll
            for (int it = 0; it < ITEMS; it++) {
                const int e = tid + it * 256;
                const int j = fc_div(e, p.divLW), lx = e - j * p.LW;
                // columns this block needs of band j
                const int lxA = (j == 0) ? tw0 * 6 : 0, lxB = (j == NB - 1) ? twL * 6 + 8 : p.LW;
                const bool need = e < items && lx >= lxA && lx < lxB;
                dstOff[it] = need ? j * 8 * p.LW + lx : -1;
                const uint32_t gb = gb0 + j;
                const uint32_t n = fc_div(gb, p.divTH), th = gb - n * p.tH;
                const int gx = lx - p.pad_l, gy0 = (int)th * 6 - p.pad_t;
                const bool colIn = need && (uint32_t)gx < (uint32_t)p.W;
                // byte offset of row gy0 (possibly above the image: then only rows that are inside are used)
                const uint32_t off0 = (n * imgStride + chanOff + (uint32_t)(gy0 * p.W + gx)) * 4u;
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const bool in = colIn && (uint32_t)(gy0 + i) < (uint32_t)p.H;
                    const uint32_t off = in ? off0 + (uint32_t)(i * p.W) * 4u : 0x80000000u;
                    d[it][i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xres, (int)off, 0, 0));
                }
            }
        } else {
#pragma unroll
            for (int it = 0; it < ITEMS; it++) {
                const int e = tid + it * 256;
                dstOff[it] = -1;
#pragma unroll
                for (int i = 0; i < 8; i++) d[it][i] = 0.f;
                if (e < items) {
                    const int j = fc_div(e, p.divLW), lx = e - j * p.LW;
                    const int lxA = (j == 0) ? tw0 * 6 : 0, lxB = (j == NB - 1) ? twL * 6 + 8 : p.LW;
                    if (lx >= lxA && lx < lxB) {
                        dstOff[it] = j * 8 * p.LW + lx;
                        const uint32_t gb = gb0 + j;
                        const uint32_t n = fc_div(gb, p.divTH), th = gb - n * p.tH;
                        const int gx = lx - p.pad_l, gy0 = (int)th * 6 - p.pad_t;
                        if (gx >= 0 && gx < p.W) {
                            const float *src = p.x + (((size_t)n * p.C + c) * p.H) * p.W + gx;
#pragma unroll
                            for (int i = 0; i < 8; i++) {
                                const int gy = gy0 + i;
                                if (gy >= 0 && gy < p.H) d[it][i] = src[(long)gy * p.W];
                            }
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int it = 0; it < ITEMS; it++) {
            if (dstOff[it] >= 0) {
                float o[8];
                bt8(d[it], o);
                float *dstl = lds + dstOff[it];
#pragma unroll
                for (int i = 0; i < 8; i++) dstl[i * p.LW] = o[i];
            }
        }
    }
    __syncthreads();

#ifdef FC_IT_VEC4
    if (TPB == 128) {
        // Pass 2, 16 bytes per plane store: thread = (row i of the tile, group of 4 consecutive tiles); B along the row
        // of each of its tiles, then one 16-byte store per column frequency: 32 lanes cover the 512 bytes a block owns
        // of a plane.
        typedef float floatx4 __attribute__((ext_vector_type(4)));
        const int g = tid & 31, i = tid >> 5;
        floatx4 o[8];
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const uint32_t t = t0 + 4 * g + q4;
            float r[8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) r[jj] = 0.f;
            if (c < p.C && t < (uint32_t)p.T) {
                const uint32_t gb = fc_div(t, p.divTW);
                const int q = t - gb * p.tW, j = gb - gb0;
                const float *row = lds + (j * 8 + i) * p.LW + q * 6;
                float d[8];
#pragma unroll
                for (int jj = 0; jj < 8; jj++) d[jj] = row[jj];
                bt8(d, r);
            }
#pragma unroll
            for (int jj = 0; jj < 8; jj++) o[jj][q4] = r[jj];
        }
        float *pf = p.V + (size_t)(i * 8) * plane + (size_t)c * p.T_pad + t0 + 4 * g;
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            *reinterpret_cast<floatx4 *>(pf) = o[jj];
            pf += plane;
        }
        return;
    }
#endif
    constexpr int IPT = 8 * TPB / 256;     // rows of the 8x8 tile per thread
    const int tl = tid % TPB;
    // rows ig*IPT .. +IPT-1 of the tile: the same for a whole wavefront when TPB is a multiple of 64
    const int igLane = tid / TPB;
    const int ig = TPB >= 64 ? __builtin_amdgcn_readfirstlane(igLane) : igLane;
    const uint32_t t = t0 + tl;
    // plane f of this block starts at V + f * plane + c * T_pad + t0; the lane adds 4 * tl
    // (with 32 tiles per block the two halves of a wavefront are on different planes: a pointer per lane)
    float *pf = p.V + (size_t)(ig * IPT * 8) * plane + (size_t)c * p.T_pad + t0;
    const uint32_t laneOff = (uint32_t)tl * 4u;
    if (c < p.C && t < (uint32_t)p.T) {
        const uint32_t gb = fc_div(t, p.divTW);
        const int q = t - gb * p.tW, j = gb - gb0;
        const float *rows = lds + (j * 8 + ig * IPT) * p.LW + q * 6;
#pragma unroll
        for (int ii = 0; ii < IPT; ii++) {
            const float *row = rows + ii * p.LW;
            float d[8], o[8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) d[jj] = row[jj];
            bt8(d, o);
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                store_at(pf, laneOff, o[jj]);
                pf += plane;       // stepped, not multiplied: a 64-bit product would be made with vector instructions
            }
        }
    } else {
        // padding channel or padding tile: the GEMM reads it, so it must be zero
#pragma unroll
        for (int ii = 0; ii < IPT * 8; ii++) {
            store_at(pf, laneOff, 0.f);
            pf += plane;
        }
    }
}

template <int TPB, int ITEMS, bool BUF>
__global__ __launch_bounds__(256) void wino_input_transform_kernel(const InTParams p) {
    extern __shared__ float lds[];   // [bands][8][LW]
    input_transform_block<TPB, ITEMS, BUF>(p, blockIdx.x, blockIdx.y, lds);
}

// Filter and input transform in one launch (the filter transform of a layer is a short
// kernel: launched by itself it costs a launch and a drain of the whole chip per layer).
// The first nFilter workgroups transform the filter, the others the input.
template <int TPB, int ITEMS, bool BUF>
__global__ __launch_bounds__(256) void wino_filter_input_transform_kernel(const FilterTParams q, const InTParams p,
                                                                          int filterGridX, int nFilter, int inputGridX) {
    extern __shared__ float lds[];
    const int b = blockIdx.x;
    if (b < nFilter) {
        const int by = b / filterGridX;
        filter_transform_block(q, b - by * filterGridX, by);
    } else {
        const int i = b - nFilter, c = i / inputGridX;
        input_transform_block<TPB, ITEMS, BUF>(p, i - c * inputGridX, c, lds);
    }
}

// ---------------------------------------------------------------- output

struct OutTParams {
    const float *M;
    const float *bias;
    float *y;
    int N, K, OH, OW, relu;
    int tH, tW;
    long T;
    int K_pad;
    long T_pad;
    fc_fastdiv divTH, divTW;
};

// Block = one output channel x TPB consecutive tiles, one thread per tile.  The 64
// plane loads of a wavefront are each 256 contiguous bytes.  The 6x6 results are
// laid into LDS as the image rows they cover, row after row exactly as in y (a
// band of a 14-row image whose tiles reach past the last row takes 2 rows, not 6),
// and copied out image by image: the bands of an image that the block covers
// completely are one contiguous run of rows*OW floats in LDS and in y (a whole
// 14x14 image leaves in one 16-byte store per lane instead of five 4-byte ones),
// a partly covered band (first or last of the range) is one run per row.
// Everything that does not depend on the lane (plane bases, band geometry of the
// copy loop) is kept in scalar registers: the kernel spends a quarter of its
// vector instructions on addresses otherwise.
// TPT: tiles per thread.  1: a lane owns one tile and loads 4 bytes per plane.  2 (a measured variant, built
// with -DFC_OT_VEC2): a lane owns two consecutive tiles and loads 8 bytes per plane, half the load instructions
// per byte for 128 more registers.
template <int TPB, int TPT = 1>
__global__ __launch_bounds__(TPB / TPT) void wino_output_transform_kernel(const OutTParams p) {
    extern __shared__ __attribute__((aligned(16))) float lds[];   // image rows of OW floats, at most 6 per band
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k = blockIdx.y;
    const uint32_t t0 = blockIdx.x * TPB;
    if (t0 >= (uint32_t)p.T) return;
    const uint32_t tLast = min((uint32_t)(t0 + TPB), (uint32_t)p.T) - 1;
    const uint32_t gb0 = fc_div(t0, p.divTW), gbL = fc_div(tLast, p.divTW);
    const int tw0 = t0 - gb0 * p.tW, twL = tLast - gbL * p.tW;
    // image rows in LDS: row (n*OH + th*6 + i) - row0 for band n*tH + th, row0 = first row of the first band
    const uint32_t n0 = fc_div(gb0, p.divTH), nL = fc_div(gbL, p.divTH);
    const int row0 = (int)n0 * p.OH + (int)(gb0 - n0 * p.tH) * 6;

    const uint32_t tFirst = t0 + TPT * tid;
    if (tFirst <= tLast) {
        const size_t plane = (size_t)p.K_pad * p.T_pad;
        const float *src = p.M + (size_t)k * p.T_pad + t0;      // uniform
        const uint32_t laneOff = (uint32_t)tid * (4u * TPT);
        float m[TPT][8][8];
        const float *pf = src;      // stepped, not multiplied: a 64-bit product would be made with vector instructions
#pragma unroll
        for (int f = 0; f < 64; f++) {
            if (TPT == 1) {
                m[0][f >> 3][f & 7] = load_m_at(pf, laneOff);
            } else {
                typedef float floatx2 __attribute__((ext_vector_type(2)));
                const floatx2 v = __builtin_nontemporal_load(reinterpret_cast<const floatx2 *>(reinterpret_cast<const char *>(pf) + laneOff));
                m[0][f >> 3][f & 7] = v[0];
                m[TPT - 1][f >> 3][f & 7] = v[1];
            }
            pf += plane;
        }
        const float b = p.bias ? p.bias[k] : 0.f;
        // ReLU as a maximum with 0, no ReLU as a maximum with -inf: one v_maximum3_f32 either way, which keeps a NaN
        const float floorv = p.relu ? 0.f : -__builtin_inff();
#pragma unroll
        for (int u = 0; u < TPT; u++) {
            const uint32_t t = tFirst + u;
            if (t > tLast) break;
            const uint32_t gb = fc_div(t, p.divTW);
            const int q = t - gb * p.tW;
            const uint32_t n = fc_div(gb, p.divTH);
            const int th = (int)(gb - n * p.tH);
            float tmp[6][8];
#pragma unroll
            for (int jj = 0; jj < 8; jj++) {
                const float col[8] = {m[u][0][jj], m[u][1][jj], m[u][2][jj], m[u][3][jj], m[u][4][jj], m[u][5][jj], m[u][6][jj], m[u][7][jj]};
                float s[6];
                at6(col, s);
#pragma unroll
                for (int i = 0; i < 6; i++) tmp[i][jj] = s[i];
            }
            float *img = lds + ((int)n * p.OH + th * 6 - row0) * p.OW + q * 6;
            const int colsLeft = p.OW - q * 6;      // columns of this tile inside the image
            const int rowsLeft = p.OH - th * 6;     // and rows: the rows below belong to the next image in LDS
#pragma unroll
            for (int i = 0; i < 6; i++) {
                // the bias goes in with element 1: at6 adds it (as m1 + m2 or m1 - m2) to each of its six outputs once
                const float row[8] = {tmp[i][0], tmp[i][1] + b, tmp[i][2], tmp[i][3], tmp[i][4], tmp[i][5], tmp[i][6], tmp[i][7]};
                float s[6];
                at6(row, s);
#pragma unroll
                for (int jj = 0; jj < 6; jj++) s[jj] = __builtin_elementwise_maximum(s[jj], floorv);
                float *dstl = img + i * p.OW;
                if (i < rowsLeft) {
                    if (colsLeft >= 6) {
#pragma unroll
                        for (int jj = 0; jj < 6; jj++) dstl[jj] = s[jj];
                    } else {
#pragma unroll
                        for (int jj = 0; jj < 6; jj++)
                            if (jj < colsLeft) dstl[jj] = s[jj];
                    }
                }
            }
        }
    }
    __syncthreads();

    constexpr int WAVES = TPB / TPT / 64;
    const size_t chan = (size_t)p.OH * p.OW;
    // one row of a partly covered band: columns xA .. xB-1 of `rows` rows
    auto copy_rows = [&](float *dst, const float *src, int rows, int xA, int xB) {
        for (int i = 0; i < rows; i++)
            for (int x = xA + lane; x < xB; x += 64) store_at(dst + i * p.OW, (uint32_t)x * 4u, src[i * p.OW + x]);
    };
    for (uint32_t n = n0 + wave; n <= nL; n += WAVES) {       // n and everything derived from it is uniform
        // bands of image n inside the block, as rows of tiles of that image
        const uint32_t gbA = max(gb0, n * p.tH), gbB = min(gbL, n * p.tH + p.tH - 1);
        const int thA = (int)(gbA - n * p.tH), thB = (int)(gbB - n * p.tH);
        // the first band of the block starts at tile tw0, its last band ends with tile twL
        const bool cutA = gbA == gb0 && tw0 > 0, cutB = gbB == gbL && (twL + 1) * 6 < p.OW;
        const bool cutBoth = cutA && cutB && gbA == gbB;      // one band, open on both sides: one copy does it
        float *img = p.y + ((size_t)n * p.K + k) * chan;
        const int simg = ((int)n * p.OH - row0) * p.OW;      // where row 0 of the image would lie in LDS
        if (cutA) {
            const int xB = (gbA == gbL) ? min((twL + 1) * 6, p.OW) : p.OW;
            copy_rows(img + thA * 6 * p.OW, lds + (simg + thA * 6 * p.OW), min(6, p.OH - thA * 6), tw0 * 6, xB);
        }
        if (cutB && !cutBoth) copy_rows(img + thB * 6 * p.OW, lds + (simg + thB * 6 * p.OW), min(6, p.OH - thB * 6), 0, (twL + 1) * 6);
        const int cA = thA + (cutA ? 1 : 0), cB = thB - (cutB ? 1 : 0);      // the bands covered completely
        if (cA <= cB) {
            const int rowA = cA * 6, rowB = min(p.OH, (cB + 1) * 6);
            const int len = (rowB - rowA) * p.OW;
            float *dst = img + rowA * p.OW;
            const float *src = lds + (simg + rowA * p.OW);
            // 16-byte pieces where the run starts on a 16-byte boundary in y and in LDS and is a whole number of them
            const bool vec4 = (len & 3) == 0 && ((((size_t)n * p.K + k) * chan + (size_t)rowA * p.OW) & 3) == 0 &&
                              ((simg + rowA * p.OW) & 3) == 0;
            if (vec4) {
                typedef float vec4f __attribute__((ext_vector_type(4)));
                for (int e = lane; e < len / 4; e += 64)
                    *reinterpret_cast<vec4f *>(reinterpret_cast<char *>(dst) + (uint32_t)e * 16u) =
                        *reinterpret_cast<const vec4f *>(reinterpret_cast<const char *>(src) + (uint32_t)e * 16u);
            } else {
                for (int e = lane; e < len; e += 64) store_at(dst, (uint32_t)e * 4u, src[e]);
            }
        }
    }
}

constexpr int kWinoMaxTilesW = 170;

// Largest of 128 / 64 / 32 tiles per block that divides the padded tile count.
int tiles_per_block(long T_pad) { return (T_pad % 128 == 0) ? 128 : (T_pad % 64 == 0) ? 64 : 32; }

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
    // output wider than 1020: a band of the input transform (8 rows x 6*tiles_w + 2 columns, two of them
    // per workgroup) no longer fits 64 KiB of LDS
    if (plan->tiles_w > kWinoMaxTilesW) return FC_ERR_UNSUPPORTED;
    if (plan->T_pad >= (1l << 31) || (size_t)plan->C_pad * plan->T_pad >= (1ull << 31) ||
        (size_t)plan->K_pad * plan->T_pad >= (1ull << 31))
        return FC_ERR_UNSUPPORTED;
    return FC_OK;
}

// Measured on MI355X (both algorithms at their best tile shape, whole-layer forward time, every 3x3
// stride-1 layer of VGG-16 and ResNet-50 at batch 1, 4 and 32, the ResNet-50 ones also at 8 and 16): with
// 16 or more input channels Winograd wins from 3.7 GFLOP of direct-convolution work on (by 1.1x to 3.2x;
// two 512-channel layers are level there); at 1.85 GFLOP the two are level (seven layers, 0.97-1.36);
// up to 0.92 GFLOP one implicit-GEMM launch, its reduction split inside the workgroups, is 1.3-2.2x ahead
// of the three launches of the staged pipeline.  The 3-channel first layer: implicit GEMM 1.5-1.7x ahead
// at batch 1 and 4, the two within 10 % at batch 32 (both bound by the stores of the output).
extern "C" int fc_prefer_winograd(const fc_conv_shape *s) {
    if (!fc_shape_ok(s) || s->kh != 3 || s->kw != 3 || s->sh != 1 || s->sw != 1) return 0;
    const int OH = fc_out_dim(s->H, s->pt, s->pb, 3, 1), OW = fc_out_dim(s->W, s->pl, s->pr, 3, 1);
    if ((OW + 5) / 6 > kWinoMaxTilesW) return 0;
    if (s->C < 16) return 0;
    const double flop = 2.0 * s->N * s->K * s->C * (double)OH * OW * 9.0;
    return flop >= 2.5e9 ? 1 : 0;
}

static int plan_check(fc_context *ctx, const fc_wino_plan *plan, const void *a, const void *b) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!plan || !a || !b) return fc_set_error(ctx, FC_ERR_INVALID, "null plan or buffer", hipSuccess);
    fc_wino_plan chk;
    const int rc = fc_wino_make_plan(&plan->shape, plan->gemm_config, &chk);
    if (rc) return fc_set_error(ctx, rc, "plan does not describe a supported layer", hipSuccess);
    if (!fc_same_wino_plan(chk, *plan))
        return fc_set_error(ctx, FC_ERR_INVALID, "plan fields were modified after fc_wino_make_plan", hipSuccess);
    return FC_OK;
}

static FilterTParams filter_params(const fc_wino_plan *plan, const float *w_dev, float *U_dev) {
    FilterTParams q;
    q.w = w_dev; q.U = U_dev;
    q.K = plan->shape.K; q.C = plan->shape.C; q.K_pad = plan->K_pad; q.C_pad = plan->C_pad;
    return q;
}

extern "C" int fc_wino_filter_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev,
                                        float *U_dev) {
    const int rc = plan_check(ctx, plan, w_dev, U_dev);
    if (rc) return rc;
    const dim3 grid((plan->K_pad + 63) / 64, (plan->C_pad + 3) / 4);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_filter_transform: too many channels", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_KERNEL_TRAN);
    wino_filter_transform_kernel<<<grid, dim3(256), 0, ctx->stream>>>(filter_params(plan, w_dev, U_dev));
    FC_LAUNCH_CHECK(ctx, "wino_filter_transform_kernel");
    return FC_OK;
}

// Input transform, alone (q == NULL) or in one launch with the filter transform.
static int launch_input_transform(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, float *V_dev,
                                  const FilterTParams *q) {
    const fc_conv_shape &s = plan->shape;
    InTParams p;
    p.x = x_dev; p.V = V_dev;
    p.N = s.N; p.C = s.C; p.H = s.H; p.W = s.W; p.pad_t = s.pt; p.pad_l = s.pl;
    p.tH = plan->tiles_h; p.tW = plan->tiles_w;
    p.T = plan->T; p.C_pad = plan->C_pad; p.T_pad = plan->T_pad;
    p.LW = 6 * p.tW + 2;
    p.divLW = fc_make_fastdiv(p.LW);
    p.divTH = fc_make_fastdiv(p.tH);
    p.divTW = fc_make_fastdiv(p.tW);
    // The largest of 128 / 64 / 32 tiles per block that divides the padded tile count and whose bands
    // fit 64 KiB of LDS (a range of tpb tiles touches at most maxBands bands of 8 rows x LW columns).
    // fc_wino_make_plan admits at most 170 tiles per band, for which 32 tiles per block always fit.
    int tpb = tiles_per_block(plan->T_pad), maxBands = 0;
    size_t ldsBytes = 0;
    for (;; tpb /= 2) {
        maxBands = (tpb + p.tW - 2) / p.tW + 1;
        ldsBytes = (size_t)maxBands * 8 * p.LW * sizeof(float);
        if (ldsBytes <= 64 * 1024 || tpb == 32) break;
    }
    if (ldsBytes > 64 * 1024) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: image too wide", hipSuccess);
    const dim3 grid((unsigned)(plan->T_pad / tpb), plan->C_pad);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: more than 65535 channels", hipSuccess);
    // columns (band x column pairs) per thread in pass 1: at most 8, since maxBands * LW <= 2048
    const int itemsPerThread = (maxBands * p.LW + 255) / 256;
    if (itemsPerThread > 8) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: image too wide", hipSuccess);
    const int filterGridX = (plan->K_pad + 63) / 64;
    const long nFilter = q ? (long)filterGridX * ((plan->C_pad + 3) / 4) : 0;
    const long total = nFilter + (long)grid.x * grid.y;
    if (total >= (1l << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_input_transform: grid too large", hipSuccess);
    const size_t xBytes = sizeof(float) * s.N * s.C * s.H * s.W;
    const bool useBuf = xBytes <= ((size_t)1 << 31);
    p.xBytes = useBuf ? (unsigned)xBytes : 0u;
    fc_stage_scope scope(ctx, FC_STAGE_INPUT_TRAN);
#define FC_LAUNCH_ONE(TPB_, ITEMS_, BUF_)                                                                                \
    do {                                                                                                                 \
        if (q)                                                                                                           \
            wino_filter_input_transform_kernel<TPB_, ITEMS_, BUF_><<<dim3((unsigned)total), dim3(256), ldsBytes, ctx->stream>>>( \
                *q, p, filterGridX, (int)nFilter, (int)grid.x);                                                          \
        else                                                                                                             \
            wino_input_transform_kernel<TPB_, ITEMS_, BUF_><<<grid, dim3(256), ldsBytes, ctx->stream>>>(p);              \
    } while (0)
    // the pointer path (inputs of more than 2 GiB) is built for 8 columns per thread only
#define FC_LAUNCH_INT(TPB_)                                        \
    do {                                                           \
        if (!useBuf) FC_LAUNCH_ONE(TPB_, 8, false);                \
        else if (itemsPerThread <= 2) FC_LAUNCH_ONE(TPB_, 2, true); \
        else if (itemsPerThread <= 4) FC_LAUNCH_ONE(TPB_, 4, true); \
        else if (itemsPerThread <= 6) FC_LAUNCH_ONE(TPB_, 6, true); \
        else FC_LAUNCH_ONE(TPB_, 8, true);                         \
    } while (0)
    if (tpb == 128) FC_LAUNCH_INT(128);
    else if (tpb == 64) FC_LAUNCH_INT(64);
    else FC_LAUNCH_INT(32);
#undef FC_LAUNCH_INT
#undef FC_LAUNCH_ONE
    FC_LAUNCH_CHECK(ctx, "wino_input_transform_kernel");
    return FC_OK;
}

extern "C" int fc_wino_input_transform(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                                       float *V_dev) {
    const int rc = plan_check(ctx, plan, x_dev, V_dev);
    if (rc) return rc;
    return launch_input_transform(ctx, plan, x_dev, V_dev, NULL);
}

extern "C" int fc_wino_filter_input_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev, float *U_dev,
                                              const float *x_dev, float *V_dev) {
    int rc = plan_check(ctx, plan, w_dev, U_dev);
    if (rc) return rc;
    rc = plan_check(ctx, plan, x_dev, V_dev);
    if (rc) return rc;
    const FilterTParams q = filter_params(plan, w_dev, U_dev);
    return launch_input_transform(ctx, plan, x_dev, V_dev, &q);
}

extern "C" int fc_wino_output_transform(fc_context *ctx, const fc_wino_plan *plan, const float *M_dev,
                                        const float *bias_dev, int relu, float *y_dev) {
    const int rc = plan_check(ctx, plan, M_dev, y_dev);
    if (rc) return rc;
    const fc_conv_shape &s = plan->shape;
    OutTParams p;
    p.M = M_dev; p.bias = bias_dev; p.y = y_dev;
    p.N = s.N; p.K = s.K; p.OH = plan->OH; p.OW = plan->OW; p.relu = relu;
    p.tH = plan->tiles_h; p.tW = plan->tiles_w;
    p.T = plan->T; p.K_pad = plan->K_pad; p.T_pad = plan->T_pad;
    p.divTH = fc_make_fastdiv(p.tH);
    p.divTW = fc_make_fastdiv(p.tW);
    int tpb = (plan->T_pad % 128 == 0 && plan->T >= 128) ? 128 : 64;
    int maxBands = (tpb + p.tW - 2) / p.tW + 1;
    size_t ldsBytes = (size_t)maxBands * 6 * p.OW * sizeof(float);
    if (ldsBytes > 64 * 1024 && tpb == 128) {
        tpb = 64;
        maxBands = (tpb + p.tW - 2) / p.tW + 1;
        ldsBytes = (size_t)maxBands * 6 * p.OW * sizeof(float);
    }
    if (ldsBytes > 64 * 1024) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_output_transform: image too wide", hipSuccess);
    const dim3 grid((unsigned)((plan->T + tpb - 1) / tpb), s.K);
    if (grid.y > 65535) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_output_transform: more than 65535 channels", hipSuccess);
    if (((uintptr_t)y_dev & 15) != 0) return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_output_transform: y must be 16-byte aligned", hipSuccess);
    fc_stage_scope scope(ctx, FC_STAGE_OUTPUT_TRAN);
#ifdef FC_OT_VEC2
    if (tpb == 128) wino_output_transform_kernel<128, 2><<<grid, dim3(64), ldsBytes, ctx->stream>>>(p);
#else
    if (tpb == 128) wino_output_transform_kernel<128><<<grid, dim3(128), ldsBytes, ctx->stream>>>(p);
#endif
    else wino_output_transform_kernel<64><<<grid, dim3(64), ldsBytes, ctx->stream>>>(p);
    FC_LAUNCH_CHECK(ctx, "wino_output_transform_kernel");
    return FC_OK;
}

extern "C" int fc_wino_forward(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, const float *w_dev,
                               const float *bias_dev, int relu, int filter_ready, float *U_dev, float *V_dev,
                               float *M_dev, float *y_dev) {
    int rc;
    if (!filter_ready && w_dev && fc_wino_prefer_raw_filter_gemm(plan)) {
        // few tiles and no transformed filter yet: the products are made from the 9 filter taps, U is not written
        rc = fc_wino_input_transform(ctx, plan, x_dev, V_dev);
        if (rc) return rc;
        rc = fc_wino_gemm_raw_filter(ctx, plan, w_dev, V_dev, M_dev, 0, 0);
        if (rc) return rc;
        return fc_wino_output_transform(ctx, plan, M_dev, bias_dev, relu, y_dev);
    }
    rc = filter_ready ? fc_wino_input_transform(ctx, plan, x_dev, V_dev)
                      : fc_wino_filter_input_transform(ctx, plan, w_dev, U_dev, x_dev, V_dev);
    if (rc) return rc;
    rc = fc_wino_gemm(ctx, plan, U_dev, V_dev, M_dev);
    if (rc) return rc;
    return fc_wino_output_transform(ctx, plan, M_dev, bias_dev, relu, y_dev);
}
