// Internal declarations shared by the HIP translation units of libfastconv_hip.
#pragma once

#include <hip/hip_runtime.h>

#include <string>
#include <vector>

#include "fastconv_hip.h"

struct fc_timing_pair {
    int stage;
    hipEvent_t start, stop;
};

struct fc_context {
    uint32_t magic;
    int device;
    hipStream_t stream;
    hipDeviceProp_t props;
    std::string last_error;
    unsigned timing_mask;   // bit s set: launches of stage s are bracketed by events
    std::vector<hipEvent_t> free_events;
    std::vector<fc_timing_pair> pending;
    double stage_ms[FC_STAGE_COUNT];
    long stage_launches[FC_STAGE_COUNT];
    // large dynamic LDS sizes are granted per kernel and per device, once per context
    bool fused_lds_granted, onepass_lds_granted, smallc_lds_granted;
    bool capturing;         // between fc_graph_begin and fc_graph_end
    // shader-clock probe: its own stream and result buffer, created on first use
    hipStream_t probe_stream;
    unsigned long long *probe_buf;
    int probe_samples;      // > 0 while a probe is running
    // device address of the static split-reduction workspace of fc_conv_implicit_gemm_static
    float *igemm_static_ws;
};

struct fc_graph {
    uint32_t magic;
    fc_context *ctx;
    hipGraph_t graph;
    hipGraphExec_t exec;
};

struct fc_pool {
    uint32_t magic;
    fc_context *ctx;
    char *base;
    size_t capacity, used, peak;
};

static const uint32_t FC_CTX_MAGIC = 0x46434358u;   // "FCCX"
static const uint32_t FC_POOL_MAGIC = 0x4643504cu;  // "FCPL"
static const uint32_t FC_GRAPH_MAGIC = 0x46434752u; // "FCGR"

int fc_set_error(fc_context *ctx, int status, const char *what, hipError_t err);
// implicit_gemm.hip: looks up the static workspace of this context's device (once per device)
int fc_igemm_static_init(fc_context *ctx);
// gives the static workspace of the context's device back when this context was the one using it
void fc_igemm_static_release(fc_context *ctx);
bool fc_ctx_ok(const fc_context *ctx);
// implicit_gemm_wavesplit.hip: the implicit-GEMM configurations whose workgroups split the reduction over their
// wavefronts (small tiles, one launch per layer, for layers with few output pixels).  `index` counts them from 0;
// their public ids follow the LDS-tiled configurations of implicit_gemm.hip.
int fc_igemm_ws_num_shapes();
void fc_igemm_ws_get_config(int index, int id, fc_gemm_config *cfg);
bool fc_igemm_ws_supports(const fc_conv_shape *s);
int fc_igemm_ws_choose(const fc_conv_shape *s, long Npix);      // index of the untuned choice, or -1
int fc_igemm_ws_pack(fc_context *ctx, const fc_igemm_plan *plan, const float *w_dev, float *Wq_dev, int32_t *table_dev);
int fc_igemm_ws_run(fc_context *ctx, const fc_igemm_plan *plan, int index, const float *x_dev, const float *Wq_dev,
                    const int32_t *table_dev, const float *bias_dev, int relu, float *y_dev, bool timed);
// wino_smallc.hip: the single-kernel Winograd path of layers with at most four input channels.
// Called by the fc_wino_*onepass* entry points after they have checked plan and pointers.
bool fc_wino_smallc_applies(const fc_conv_shape *s);
int fc_wino_smallc_filter_transform(fc_context *ctx, const fc_wino_plan *plan, const float *w_dev, float *U_dev);
// w_dev == nullptr: U_dev holds the transformed filter; otherwise the kernel transforms w_dev itself and fills U_dev
int fc_wino_smallc_conv(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev, float *U_dev, const float *w_dev,
                        const float *bias_dev, int relu, float *y_dev);
// whether a forward call that has to transform the filter should leave that to the convolution kernel
bool fc_wino_smallc_transforms_inside(const fc_context *ctx, const fc_wino_plan *plan);

// Brackets one kernel launch with events when timing is on.
struct fc_stage_scope {
    fc_context *ctx;
    hipEvent_t stop;
    bool active;
    fc_stage_scope(fc_context *c, int stage);
    ~fc_stage_scope();
};

#define FC_HIP_CHECK(ctx, expr)                                              \
    do {                                                                     \
        hipError_t e__ = (expr);                                             \
        if (e__ != hipSuccess) return fc_set_error((ctx), FC_ERR_HIP, #expr, e__); \
    } while (0)

#define FC_LAUNCH_CHECK(ctx, name)                                           \
    do {                                                                     \
        hipError_t e__ = hipGetLastError();                                  \
        if (e__ != hipSuccess) return fc_set_error((ctx), FC_ERR_HIP, name, e__); \
    } while (0)

static inline long fc_round_up(long v, long m) { return (v + m - 1) / m * m; }

static inline int fc_out_dim(int in, int pa, int pb, int k, int s) { return (in + pa + pb - k) / s + 1; }

static inline bool fc_shape_ok(const fc_conv_shape *s) {
    if (!s) return false;
    if (s->N <= 0 || s->C <= 0 || s->H <= 0 || s->W <= 0 || s->K <= 0) return false;
    if (s->kh <= 0 || s->kw <= 0 || s->sh <= 0 || s->sw <= 0) return false;
    if (s->pt < 0 || s->pb < 0 || s->pl < 0 || s->pr < 0) return false;
    if (s->H + s->pt + s->pb < s->kh || s->W + s->pl + s->pr < s->kw) return false;
    return true;
}

static inline bool fc_same_shape(const fc_conv_shape &a, const fc_conv_shape &b) {
    return a.N == b.N && a.C == b.C && a.H == b.H && a.W == b.W && a.K == b.K && a.kh == b.kh && a.kw == b.kw &&
           a.sh == b.sh && a.sw == b.sw && a.pt == b.pt && a.pb == b.pb && a.pl == b.pl && a.pr == b.pr;
}

// Every field of a plan a caller hands in is compared with the plan the library itself makes
// for the same shape and configuration: the kernels take their sizes from it unverified.
static inline bool fc_same_wino_plan(const fc_wino_plan &a, const fc_wino_plan &b) {
    return fc_same_shape(a.shape, b.shape) && a.OH == b.OH && a.OW == b.OW && a.tiles_h == b.tiles_h &&
           a.tiles_w == b.tiles_w && a.T == b.T && a.K_pad == b.K_pad && a.C_pad == b.C_pad && a.T_pad == b.T_pad &&
           a.gemm_config == b.gemm_config && a.U_bytes == b.U_bytes && a.V_bytes == b.V_bytes && a.M_bytes == b.M_bytes;
}

static inline bool fc_same_igemm_plan(const fc_igemm_plan &a, const fc_igemm_plan &b) {
    return fc_same_shape(a.shape, b.shape) && a.OH == b.OH && a.OW == b.OW && a.Kred == b.Kred &&
           a.Kred_pad == b.Kred_pad && a.K_pad == b.K_pad && a.Npix == b.Npix && a.config == b.config &&
           a.Wp_bytes == b.Wp_bytes && a.table_bytes == b.table_bytes && a.split_k == b.split_k &&
           a.ws_bytes == b.ws_bytes;
}

// Unsigned division by a runtime constant: q = (n * mul) >> (32 + shift), exact
// for n < 2^31 (round-up method with a 33-bit multiplier folded by one add).
struct fc_fastdiv {
    uint32_t mul, shift, div;
};

static inline fc_fastdiv fc_make_fastdiv(uint32_t d) {
    fc_fastdiv f;
    f.div = d;
    if (d == 1) { f.mul = 0; f.shift = 0; return f; }
    uint32_t l = 0;
    while ((1ull << l) < d) l++;
    // magic = ceil(2^(32+l) / d) - 2^32, fits 32 bits
    const uint64_t m = ((1ull << 32) * ((1ull << l) - d)) / d + 1;
    f.mul = (uint32_t)m;
    f.shift = l;
    return f;
}

__device__ __forceinline__ uint32_t fc_div(uint32_t n, const fc_fastdiv f) {
    if (f.div == 1) return n;
    const uint32_t t = __umulhi(n, f.mul);
    return (t + ((n - t) >> 1)) >> (f.shift - 1);
}

// A pointer that is the same for every lane, pinned to scalar registers: without the pin the
// compiler turns a uniform base that advances in a loop into a 64-bit pointer per lane and pays
// a vector add per access.
template <class T>
__device__ __forceinline__ T *uniform_ptr(T *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    // through a global-memory pointer type: rebuilt from an integer the pointer would otherwise be a generic one
    typedef __attribute__((address_space(1))) T GlobalT;
    return (T *)reinterpret_cast<GlobalT *>(((uint64_t)hi << 32) | lo);
}

