// Winograd F(6,3) for layers with at most four input channels (the RGB layer in front of a
// network): the whole layer in one kernel on the vector ALUs.  With so few channels the 64
// per-frequency products are C multiply-adds each, less work than the output transform that
// follows them, so there is nothing for the matrix cores to do and the layer is bound by the
// stores of y.  A lane owns one tile: it keeps the products of one tile column in registers and
// turns them into outputs without any exchange between lanes.  A workgroup transforms the patches
// of its tiles into LDS once (V, never in HBM); each of its four wavefronts then walks over its
// share of the output channels, one per step, taking the transformed filter of the channel from a
// register (one frequency per lane) and storing the outputs of the channel before, row by row,
// between the columns of the current one.
// Same mathematics as winoF63ZC/winoF63ZC.cpp:433-973; the reference has no counterpart of the
// specialisation (its blocked pipeline, winoF63/winoF63.cpp:975-1750, runs every layer).
#include <hip/hip_runtime.h>

#include "fc_internal.h"
#include "wino_math.h"

namespace {

constexpr int kScThreads = 256;
constexpr int kScStageFloats = 64 * 6;   // per wavefront: one output row of its 64 tiles

// Tiles per workgroup, one per lane.  With three channels 62 of the 64 lanes are used: V
// (62 x 64 x 3 floats) and the four store buffers then take 53760 bytes, a third of a CU's LDS,
// and three workgroups share a CU.
__host__ __device__ constexpr int sc_tiles(int C) { return C == 3 ? 62 : 64; }

struct SmallCParams {
    int N, H, W, K, K_pad, OH, OW, pad_t, pad_l, tH, tW;
    long T;
    unsigned xBytes; // size of x, at most 2^31
    int tileBlocks, blocksPerXcd;
    int kPerBlock;   // output channels per workgroup: 64, 16 or 8 (a multiple of 8)
    int relu;
    int zero;        // always 0
    fc_fastdiv divTW, divTH;
};

// Filter transform into Us[K_pad][8 j][8 i][4 c]: the 32 values a wavefront needs for one tile
// column j of one output channel are 128 contiguous bytes.  Channels C..3 and output channels
// K..K_pad-1 are zero.
__global__ __launch_bounds__(256) void wino_smallc_filter_kernel(const float *__restrict__ w, float *__restrict__ U,
                                                                 int K, int C, int K_pad) {
    const int id = blockIdx.x * 256 + threadIdx.x;
    const int k = id >> 2, c = id & 3;
    if (k >= K_pad) return;
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
    float *dst = U + (size_t)k * 256 + c;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float o[8];
        g8(t[i], o);
#pragma unroll
        for (int j = 0; j < 8; j++) dst[(j * 8 + i) * 4] = o[j];
    }
}

// The transformed filter of one output channel, one frequency per lane: lane f = 8 j + i holds
// U[k][i][j][0..C-1].  A product takes its filter value from there with v_readlane (one more
// vector instruction per multiply-add, but no memory access inside the loop: scalar loads issued a
// column ahead waited for the L2 behind the kernel's own stores).
template <int C>
struct UReg {
    float c[C];
};

template <int C>
__device__ __forceinline__ UReg<C> load_ureg(const float *__restrict__ U, int k, int lane) {
    UReg<C> r;
    const float *src = U + (size_t)k * 256 + lane * 4;
#pragma unroll
    for (int c = 0; c < C; c++) r.c[c] = src[c];
    return r;
}

// The same operand made from the 3x3 filter inside the convolution kernel (no filter-transform launch in front
// of a layer with few tiles).  load_raw: lane e < 9*C fetches value e of the 9*C filter values of channel k
// (zeros past the last channel).  make_ureg: lane f = 8 j + i turns them into U[k][i][j][c] = (G g G^T)[i][j];
// row i of G applied as g8 applies it, ((a0*g0 + a2*g2) + a1*g1) * scale with coefficients 0, +-1, +-2, 4 whose
// products are exact (what differs from wino_smallc_filter_kernel's values is where the compiler fuses a scale
// into the addition that follows it: the last bit of some values).
template <int C>
__device__ __forceinline__ float load_raw(const float *__restrict__ w, int K, int k, int lane) {
    const float *src = uniform_ptr(w + (size_t)min(k, K - 1) * (9 * C));
    const float v = src[min(lane, 9 * C - 1)];
    return (k < K && lane < 9 * C) ? v : 0.f;
}

struct GRow {
    float a0, a2, a1, scale;
};

__device__ __forceinline__ GRow g_row(int i) {
    const float c29 = (float)(-2.0 / 9), c90 = (float)(1.0 / 90), c180 = (float)(1.0 / 180);
    GRow r;
    r.a0 = i == 7 ? 0.f : (i == 5 || i == 6) ? 4.f : 1.f;
    r.a2 = i == 0 ? 0.f : (i == 3 || i == 4) ? 4.f : 1.f;
    r.a1 = (i == 0 || i == 7) ? 0.f : i == 1 ? 1.f : i == 2 ? -1.f : (i & 1) ? 2.f : -2.f;
    r.scale = (i == 0 || i == 7) ? 1.f : i <= 2 ? c29 : i <= 4 ? c90 : c180;
    return r;
}

__device__ __forceinline__ float g_apply(const GRow &r, float g0, float g1, float g2) {
    return ((r.a0 * g0 + r.a2 * g2) + r.a1 * g1) * r.scale;
}

template <int C>
__device__ __forceinline__ UReg<C> make_ureg(float raw, const GRow &gi, const GRow &gj) {
    UReg<C> r;
#pragma unroll
    for (int c = 0; c < C; c++) {
        float g[9];
#pragma unroll
        for (int e = 0; e < 9; e++) g[e] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, raw), c * 9 + e));
        float t[3];
#pragma unroll
        for (int b = 0; b < 3; b++) t[b] = g_apply(gi, g[b], g[3 + b], g[6 + b]);      // column b of the filter: rows 0, 1, 2
        r.c[c] = g_apply(gj, t[0], t[1], t[2]);
    }
    return r;
}

// One tile column of one output channel: the eight products over the input channels and the
// column half of the output transform.  The empty asm ties the results to this point of the
// instruction stream (pure arithmetic is otherwise free to sink below the scheduling barrier
// that follows, which leaves every operand loaded so far alive).
template <int C>
__device__ __forceinline__ void column_products(const UReg<C> &u, const float (&v)[8][C], float (&r)[6][8], int j) {
    float m[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        float a = 0.f;
#pragma unroll
        for (int c = 0; c < C; c++) {
            const float uf = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, u.c[c]), j * 8 + i));
            a = c == 0 ? uf * v[i][0] : fmaf(uf, v[i][c], a);
        }
        m[i] = a;
    }
    float s[6];
    at6(m, s);
    asm volatile("" : "+v"(s[0]), "+v"(s[1]), "+v"(s[2]), "+v"(s[3]), "+v"(s[4]), "+v"(s[5]));
#pragma unroll
    for (int q = 0; q < 6; q++) r[q][j] = s[q];
}

// Orders the LDS accesses of the lanes of one wavefront: the hardware executes a wavefront's LDS
// instructions in order, so no instruction is needed, but the compiler must not move, merge or
// drop them across this point (without it, it treats a lane's stores that the same lane never
// reads back as dead).
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// What a lane needs to store its outputs.  Row stores: a row of the wavefront's tiles (6 floats
// per lane) is written to the wavefront's LDS buffer and read back as pairs of floats in memory
// order, so that a store instruction covers 512 contiguous bytes instead of 64 pieces of 8; pair
// i * 64 + lane belongs to tile (i * 64 + lane) / 3, its offset in y and its number of valid
// rows are fixed per lane.  Otherwise every lane stores its own 6 x 6 block.
struct ScStore {
    float *stage;        // this wavefront's LDS buffer
    uint32_t soff[3];
    int srows[3];
    float *ytile;        // first output of the lane's own tile in channel 0
    int nRows, nCols;
};

// One step of the loop over a wavefront's output channels: the eight tile columns of channel
// kcur (products over the input channels and the column half of the output transform, into rc)
// and, spread between them, the six output rows of the channel before it (row half of the output
// transform of rp, bias, ReLU, stores).  Stores issued in one burst per channel would fill the
// memory pipeline's queue and stall every wavefront of the CU at the same point of the loop; one
// row after each column keeps stores and arithmetic going side by side.  The transformed patch
// is read from LDS per channel, one column ahead of its use.
template <int C, bool ROWST, bool CUR, bool PREV>
__device__ __forceinline__ void sc_step(const SmallCParams &p, const UReg<C> &u, const float *__restrict__ bias,
                                        float *__restrict__ y, const float *vbase, const ScStore &st, int lane,
                                        int kprev, int tie, float floorv, float (&rc)[6][8], const float (&rp)[6][8]) {
    constexpr int TILES = sc_tiles(C);
    float vn[8][C];
    if (CUR) {
#pragma unroll
        for (int i = 0; i < 8; i++)
#pragma unroll
            for (int c = 0; c < C; c++) vn[i][c] = vbase[i * TILES * C + c];
    }
    const float bv = (PREV && bias) ? bias[kprev] : 0.f;
    const size_t chanStride = (size_t)p.OH * p.OW;
    float *yk = y + (size_t)(PREV ? kprev : 0) * chanStride;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        if (CUR) {
            float v[8][C];
#pragma unroll
            for (int i = 0; i < 8; i++)
#pragma unroll
                for (int c = 0; c < C; c++) v[i][c] = vn[i][c];
            if (j < 7) {
#pragma unroll
                for (int i = 0; i < 8; i++)
#pragma unroll
                    for (int c = 0; c < C; c++) vn[i][c] = vbase[((j + 1) * 8 + i) * TILES * C + c];
            }
            column_products<C>(u, v, rc, j);
        }
        if (PREV && j >= 1 && j <= 6) {
            const int q = j - 1;
            // the bias goes in with element 1: the row transform adds it (as m1 + m2 or m1 - m2) to each of its six outputs once
            const float mrow[8] = {rp[q][0], rp[q][1] + bv, rp[q][2], rp[q][3], rp[q][4], rp[q][5], rp[q][6], rp[q][7]};
            float o[6];
            at6(mrow, o);
#pragma unroll
            for (int s = 0; s < 6; s++) o[s] = __builtin_elementwise_maximum(o[s], floorv);
            if (ROWST) {
                float2 *sw = reinterpret_cast<float2 *>(st.stage) + lane * 3;
                wave_sync();   // the previous row has been read by every lane
                sw[0] = make_float2(o[0], o[1]);
                sw[1] = make_float2(o[2], o[3]);
                sw[2] = make_float2(o[4], o[5]);
                wave_sync();   // lanes read what other lanes wrote
                const float2 *ld = reinterpret_cast<const float2 *>(st.stage) + lane;
                const float2 a0 = ld[0], a1 = ld[64], a2 = ld[128];
                float *yrow = yk + (size_t)q * p.OW;
                // the conditions are recomputed per channel (tie is 0): kept across the loop they
                // would hold a pair of scalar registers each
                if (q < st.srows[0] + tie) *reinterpret_cast<float2 *>(yrow + st.soff[0]) = a0;
                if (q < st.srows[1] + tie) *reinterpret_cast<float2 *>(yrow + st.soff[1]) = a1;
                if (q < st.srows[2] + tie) *reinterpret_cast<float2 *>(yrow + st.soff[2]) = a2;
            } else if (q < st.nRows + tie) {
                float *row = st.ytile + (size_t)kprev * chanStride + (size_t)q * p.OW;
#pragma unroll
                for (int s = 0; s < 6; s++)
                    if (s < st.nCols + tie) row[s] = o[s];
            }
        }
        __builtin_amdgcn_sched_barrier(0);
    }
}

// RAWW: U_or_w is the untransformed filter [K][C][3][3]; every wavefront transforms the filters of its output
// channels itself (a few dozen vector instructions per channel), and the workgroups of the first tile block
// write them to Uout in the layout of wino_smallc_filter_kernel, so that U is filled as after that kernel.
template <int C, bool ROWST, bool RAWW>
__global__ __launch_bounds__(kScThreads) void wino_smallc_kernel(const float *__restrict__ x, const float *__restrict__ U_or_w,
                                                                 float *__restrict__ Uout, const float *__restrict__ bias,
                                                                 float *__restrict__ y, const SmallCParams p) {
    constexpr int TILES = sc_tiles(C);
    extern __shared__ float Vs[];   // [8 j][8 i][TILES][C], then one store buffer per wavefront
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const float *U = U_or_w;
    // workgroups are dealt to the eight XCDs in turn: give each XCD a contiguous range of tile
    // blocks, so that the cache lines two neighbouring blocks share meet in one L2
    const int tblk = (blockIdx.x & 7) * p.blocksPerXcd + (blockIdx.x >> 3);
    if (tblk >= p.tileBlocks) return;
    const long tl = (long)tblk * TILES + lane;
    const bool live = lane < TILES && tl < p.T;
    const uint32_t t = live ? (uint32_t)tl : 0u;
    const uint32_t band = fc_div(t, p.divTW);             // n * tH + th
    const int tw = (int)(t - band * (uint32_t)p.tW);
    const uint32_t n = fc_div(band, p.divTH);
    const int th = (int)(band - n * (uint32_t)p.tH);
    const int vlane = min(lane, TILES - 1);
    const int kpw = p.kPerBlock >> 2;
    const int kFirst = blockIdx.y * p.kPerBlock + wave * kpw;
    // RAWW: the filters of this wavefront's first two channels, asked for before anything else
    float rawA = 0.f, rawB = 0.f;
    if (RAWW) {
        rawA = load_raw<C>(U_or_w, p.K, kFirst, lane);
        rawB = load_raw<C>(U_or_w, p.K, kFirst + 1, lane);
    }

    // ---- input transform of channel `wave` of this lane's tile.  The patch is read through a
    // buffer resource: an element outside the image gets an offset past the end of x and the
    // hardware returns zero for it, so all 64 loads are in flight together and no lane branches.
    if (wave < C && lane < TILES) {
        __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(x), 0, (int)p.xBytes, 0x00020000);
        const uint32_t plane = (uint32_t)(n * C + wave) * (uint32_t)(p.H * p.W);
        const int gy0 = th * 6 - p.pad_t, gx0 = tw * 6 - p.pad_l;
        uint32_t rowOff[8];
#pragma unroll
        for (int a = 0; a < 8; a++) {
            const int gy = gy0 + a;
            rowOff[a] = (live && gy >= 0 && gy < p.H) ? (plane + (uint32_t)(gy * p.W)) * 4u : 0x80000000u;
        }
        float tmp[8][8];   // tmp[i][b] = sum_a Bt[i][a] d[a][b]
#pragma unroll
        for (int b = 0; b < 8; b++) {
            const int gx = gx0 + b;
            const bool colIn = gx >= 0 && gx < p.W;
            float d[8];
#pragma unroll
            for (int a = 0; a < 8; a++) {
                // a column inside the image is not negative, so adding it cannot clear bit 31 of a row outside
                const uint32_t off = colIn ? rowOff[a] + (uint32_t)(gx * 4) : 0x80000000u;
                d[a] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xres, (int)off, 0, 0));
            }
            float o[8];
            bt8(d, o);
#pragma unroll
            for (int i = 0; i < 8; i++) tmp[i][b] = o[i];
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float o[8];
            bt8(tmp[i], o);
#pragma unroll
            for (int j = 0; j < 8; j++) Vs[((j * 8 + i) * TILES + lane) * C + wave] = o[j];
        }
    }
    __syncthreads();

    // ---- products and output transform: this wavefront's output channels, one per step; the
    // outputs of a channel are finished and stored during the step of the next one.  (p.zero is
    // 0: it ties the LDS addresses to the loop counter, or all 64 x C values of the transformed
    // patch would be kept in registers across the loop.)
    const int kCount = min(kpw, p.K - kFirst);
    const GRow gi = g_row(lane & 7), gj = g_row(lane >> 3);
    // RAWW, first tile block: row k of U as wino_smallc_filter_kernel lays it out, [8 j][8 i][4 c]; channels C..3 and
    // the rows of the padding K..K_pad-1 are zeros
    auto keep = [&](int k, const UReg<C> &u) {
        if (RAWW && tblk == 0 && k < kFirst + kpw) {
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            v.x = u.c[0];
            if (C > 1) v.y = u.c[C > 1 ? 1 : 0];
            if (C > 2) v.z = u.c[C > 2 ? 2 : 0];
            if (C > 3) v.w = u.c[C > 3 ? 3 : 0];
            *reinterpret_cast<float4 *>(Uout + (size_t)k * 256 + lane * 4) = v;
        }
    };
    if (RAWW && tblk == 0)
        for (int k = kFirst + max(kCount, 0); k < kFirst + kpw; k++)
            *reinterpret_cast<float4 *>(Uout + (size_t)k * 256 + lane * 4) = make_float4(0.f, 0.f, 0.f, 0.f);
    if (kCount <= 0) return;
    // ReLU as a maximum with 0, no ReLU as a maximum with -inf: one v_maximum3_f32 either way, which keeps a NaN
    const float floorv = p.relu ? 0.f : -__builtin_inff();
    ScStore st;
    st.stage = Vs + 64 * TILES * C + wave * kScStageFloats;
    st.ytile = y + (size_t)n * p.K * p.OH * p.OW + (size_t)(th * 6) * p.OW + tw * 6;
    st.nRows = live ? min(6, p.OH - th * 6) : 0;
    st.nCols = min(6, p.OW - tw * 6);
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const int e2 = i * 64 + lane;
        const int le = e2 / 3, sp = e2 - 3 * le;
        const long t2l = (long)tblk * TILES + le;
        const bool ok = le < TILES && t2l < p.T;
        const uint32_t t2 = ok ? (uint32_t)t2l : 0u;
        const uint32_t band2 = fc_div(t2, p.divTW);
        const int tw2 = (int)(t2 - band2 * (uint32_t)p.tW);
        const uint32_t n2 = fc_div(band2, p.divTH);
        const int th2 = (int)(band2 - n2 * (uint32_t)p.tH);
        const int col = tw2 * 6 + 2 * sp;
        st.soff[i] = (uint32_t)(((size_t)n2 * p.K * p.OH + (size_t)th2 * 6) * p.OW + col);
        st.srows[i] = (ok && col < p.OW) ? min(6, p.OH - th2 * 6) : 0;
    }
    const float *vlanep = Vs + vlane * C;
    const int kMax = p.K_pad - 1;   // the filter of a channel is fetched one step ahead; never past the padded end
    float ra[6][8], rb[6][8];
    // the operand of channel k: from U, or (RAWW) from the filter values fetched two channels ahead, whose register
    // then takes the values of the channel two further on
    auto operand = [&](int k, float &raw) {
        if (RAWW) {
            const UReg<C> u = make_ureg<C>(raw, gi, gj);
            raw = load_raw<C>(U_or_w, p.K, k + 2, lane);
            if (k < p.K) keep(k, u);
            return u;
        }
        return load_ureg<C>(U, min(k, kMax), lane);
    };
    UReg<C> ua = operand(kFirst, rawA), ub = operand(kFirst + 1, rawB);
    sc_step<C, ROWST, true, false>(p, ua, bias, y, vlanep, st, lane, 0, 0, floorv, ra, rb);
    int kk = 1;
    for (; kk + 1 < kCount; kk += 2) {
        const int tie = kk * p.zero, tie2 = (kk + 1) * p.zero;   // one per step: equal addresses would be read once
        const int k = __builtin_amdgcn_readfirstlane(kFirst + kk);
        ua = operand(k + 1, rawA);
        sc_step<C, ROWST, true, true>(p, ub, bias, y, vlanep + tie, st, lane, k - 1, tie, floorv, rb, ra);
        ub = operand(k + 2, rawB);
        sc_step<C, ROWST, true, true>(p, ua, bias, y, vlanep + tie2, st, lane, k, tie2, floorv, ra, rb);
    }
    const int kLast = __builtin_amdgcn_readfirstlane(kFirst + kCount - 1);
    if (kk < kCount) {
        sc_step<C, ROWST, true, true>(p, ub, bias, y, vlanep, st, lane, kLast - 1, 0, floorv, rb, ra);
        sc_step<C, ROWST, false, true>(p, ua, bias, y, vlanep, st, lane, kLast, 0, floorv, ra, rb);
    } else {
        sc_step<C, ROWST, false, true>(p, ua, bias, y, vlanep, st, lane, kLast, 0, floorv, rb, ra);
    }
}

}  // namespace

// x is addressed with 32-bit byte offsets whose top bit marks "outside the image"
bool fc_wino_smallc_applies(const fc_conv_shape *s) {
    return s->C <= 4 && sizeof(float) * s->N * s->C * s->H * s->W <= ((size_t)1 << 31);
}

int fc_wino_smallc_filter_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev, float *U_dev) {
    const int threads = plan->K_pad * 4;
    fc_stage_scope scope(ctx, FC_STAGE_KERNEL_TRAN);
    wino_smallc_filter_kernel<<<dim3((threads + 255) / 256), dim3(256), 0, ctx->stream>>>(w_dev, U_dev, plan->shape.K,
                                                                                         plan->shape.C, plan->K_pad);
    FC_LAUNCH_CHECK(ctx, "wino_smallc_filter_kernel");
    return FC_OK;
}

// Output channels per workgroup: 64 when that still gives every CU a few workgroups, else 16, or 8 when even
// that leaves CUs without one (batch 1)
static int sc_k_per_block(const fc_context *ctx, const fc_wino_plan *plan) {
    const int tiles = sc_tiles(plan->shape.C);
    const long tileBlocks = (plan->T + tiles - 1) / tiles;
    const long cus = ctx->props.multiProcessorCount;
    return tileBlocks * (plan->K_pad / 64) >= 2 * cus ? 64 : tileBlocks * (plan->K_pad / 16) >= cus ? 16 : 8;
}

// Where a wavefront has only a few output channels the filter transform is cheaper inside the convolution kernel
// than as a launch in front of it (4.5 us plus the gap between two launches; the whole layer takes 13 us at batch 1).
bool fc_wino_smallc_transforms_inside(const fc_context *ctx, const fc_wino_plan *plan) {
    return sc_k_per_block(ctx, plan) < 64 && ((size_t)plan->shape.K * plan->shape.C * 9) < ((size_t)1 << 29);
}

// w_dev == nullptr: U_dev holds the transformed filter.  Otherwise the kernel transforms w_dev itself and fills U_dev.
int fc_wino_smallc_conv(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, float *U_dev, const float *w_dev,
                        const float *bias_dev, int relu, float *y_dev) {
    const fc_conv_shape &s = plan->shape;
    SmallCParams p;
    p.N = s.N; p.H = s.H; p.W = s.W; p.K = s.K; p.K_pad = plan->K_pad; p.OH = plan->OH; p.OW = plan->OW;
    p.pad_t = s.pt; p.pad_l = s.pl; p.tH = plan->tiles_h; p.tW = plan->tiles_w;
    p.T = plan->T;
    p.relu = relu;
    p.zero = 0;
    p.xBytes = (unsigned)(sizeof(float) * s.N * s.C * s.H * s.W);
    p.divTW = fc_make_fastdiv(p.tW);
    p.divTH = fc_make_fastdiv(p.tH);
    const int tiles = sc_tiles(s.C);
    const long tileBlocks = (plan->T + tiles - 1) / tiles;
    p.kPerBlock = sc_k_per_block(ctx, plan);
    const long gy = plan->K_pad / p.kPerBlock;
    if (tileBlocks >= (1l << 31) - 8 || gy > 65535)
        return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_wino_conv_onepass: grid too large", hipSuccess);
    p.tileBlocks = (int)tileBlocks;
    p.blocksPerXcd = (int)((tileBlocks + 7) / 8);
    const dim3 grid((unsigned)(p.blocksPerXcd * 8), (unsigned)gy);
    const size_t lds = sizeof(float) * (64 * tiles * s.C + (kScThreads / 64) * kScStageFloats);
    // row stores need an even output width (pairs of floats, 8-byte aligned) and 32-bit offsets into y
    const bool rowStores = (plan->OW & 1) == 0 && (size_t)s.N * s.K * plan->OH * plan->OW < ((size_t)1 << 30) &&
                  ((uintptr_t)y_dev & 7) == 0;
    if (lds > 64 * 1024 && !ctx->smallc_lds_granted) {   // four channels: 70 KiB
        if (ctx->capturing)
            return fc_set_error(ctx, FC_ERR_STATE, "fc_wino_conv_onepass: run this kernel once before recording a graph with it", hipSuccess);
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_smallc_kernel<4, true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_smallc_kernel<4, false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_smallc_kernel<4, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        FC_HIP_CHECK(ctx, hipFuncSetAttribute((const void *)wino_smallc_kernel<4, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        ctx->smallc_lds_granted = true;
    }
    fc_stage_scope scope(ctx, FC_STAGE_ONEPASS);
#define FC_SC_LAUNCH2(C_, ROWST_)                                                                                \
    do {                                                                                                         \
        if (w_dev)                                                                                               \
            wino_smallc_kernel<C_, ROWST_, true><<<grid, dim3(kScThreads), lds, ctx->stream>>>(x_dev, w_dev, U_dev, bias_dev, y_dev, p);   \
        else                                                                                                     \
            wino_smallc_kernel<C_, ROWST_, false><<<grid, dim3(kScThreads), lds, ctx->stream>>>(x_dev, U_dev, nullptr, bias_dev, y_dev, p); \
    } while (0)
#define FC_SC_LAUNCH(C_)                                                                                         \
    do {                                                                                                         \
        if (rowStores) FC_SC_LAUNCH2(C_, true);                                                                  \
        else FC_SC_LAUNCH2(C_, false);                                                                           \
    } while (0)
    switch (s.C) {
    case 1: FC_SC_LAUNCH(1); break;
    case 2: FC_SC_LAUNCH(2); break;
    case 3: FC_SC_LAUNCH(3); break;
    case 4: FC_SC_LAUNCH(4); break;
    default: return fc_set_error(ctx, FC_ERR_INVALID, "fc_wino_conv_onepass: more than four input channels", hipSuccess);
    }
#undef FC_SC_LAUNCH
#undef FC_SC_LAUNCH2
    FC_LAUNCH_CHECK(ctx, "wino_smallc_kernel");
    return FC_OK;
}
