// Context, memory arena, host<->device copies and stage timing of
// libfastconv_hip.  No compute lives here.
#include <cstdio>
#include <cstring>
#include <new>

#include "fc_internal.h"
#include "../host/utility/rng.h"

extern "C" int fc_host_fill_uniform(uint64_t seed, float lo, float hi, float *dst_host, size_t n) {
    if (!dst_host && n) return FC_ERR_INVALID;
    fastconv::FillUniform(seed, lo, hi, dst_host, n);
    return FC_OK;
}

extern "C" int fc_host_fill_normal(uint64_t seed, float sigma, float *dst_host, size_t n) {
    if (!dst_host && n) return FC_ERR_INVALID;
    fastconv::FillNormal(seed, sigma, dst_host, n);
    return FC_OK;
}

int fc_set_error(fc_context *ctx, int status, const char *what, hipError_t err) {
    if (ctx) {
        char buf[512];
        if (err != hipSuccess)
            snprintf(buf, sizeof buf, "%s: %s (%s)", fc_status_string(status), what, hipGetErrorString(err));
        else
            snprintf(buf, sizeof buf, "%s: %s", fc_status_string(status), what);
        ctx->last_error = buf;
    }
    return status;
}

bool fc_ctx_ok(const fc_context *ctx) { return ctx && ctx->magic == FC_CTX_MAGIC; }

extern "C" const char *fc_status_string(int status) {
    switch (status) {
        case FC_OK: return "ok";
        case FC_ERR_INVALID: return "invalid argument";
        case FC_ERR_NO_DEVICE: return "no usable GPU";
        case FC_ERR_HIP: return "HIP runtime error";
        case FC_ERR_OOM: return "out of device memory";
        case FC_ERR_STATE: return "wrong call order";
        case FC_ERR_UNSUPPORTED: return "size not supported";
        default: return "unknown status";
    }
}

extern "C" int fc_init(int device, fc_context **out) {
    if (!out) return FC_ERR_INVALID;
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return FC_ERR_NO_DEVICE;
    }
    if (device < 0 || device >= count) return FC_ERR_INVALID;
    if (hipSetDevice(device) != hipSuccess) return FC_ERR_NO_DEVICE;
    fc_context *ctx = new (std::nothrow) fc_context();
    if (!ctx) return FC_ERR_OOM;
    ctx->magic = FC_CTX_MAGIC;
    ctx->device = device;
    ctx->timing_mask = 0;
    ctx->fused_lds_granted = ctx->onepass_lds_granted = ctx->smallc_lds_granted = false;
    ctx->capturing = false;
    ctx->stream = nullptr;
    ctx->probe_stream = nullptr;
    ctx->probe_buf = nullptr;
    ctx->probe_samples = 0;
    memset(ctx->stage_ms, 0, sizeof ctx->stage_ms);
    memset(ctx->stage_launches, 0, sizeof ctx->stage_launches);
    if (hipGetDeviceProperties(&ctx->props, device) != hipSuccess) { delete ctx; return FC_ERR_NO_DEVICE; }
    if (strncmp(ctx->props.gcnArchName, "gfx950", 6) != 0) {
        fprintf(stderr, "fastconv: device %d is %s; this library holds gfx950 code only\n", device,
                ctx->props.gcnArchName);
        delete ctx;
        return FC_ERR_NO_DEVICE;
    }
    if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) { delete ctx; return FC_ERR_HIP; }
    ctx->igemm_static_ws = nullptr;
    if (fc_igemm_static_init(ctx) != FC_OK) {
        fprintf(stderr, "fastconv: %s\n", ctx->last_error.c_str());
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return FC_ERR_HIP;
    }
    *out = ctx;
    return FC_OK;
}

extern "C" int fc_destroy(fc_context *ctx) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    for (auto &p : ctx->pending) { (void)hipEventDestroy(p.start); (void)hipEventDestroy(p.stop); }
    for (auto &ev : ctx->free_events) (void)hipEventDestroy(ev);
    if (ctx->probe_stream) {
        (void)hipStreamSynchronize(ctx->probe_stream);
        (void)hipStreamDestroy(ctx->probe_stream);
    }
    if (ctx->probe_buf) (void)hipFree(ctx->probe_buf);
    (void)hipStreamDestroy(ctx->stream);
    fc_igemm_static_release(ctx);
    ctx->magic = 0;
    delete ctx;
    return FC_OK;
}

// One lane: per sample, wait on the constant 100 MHz counter and record both counters' advance.
// The wait is bounded twice: by the real-time counter, and by a cap on the number of polls.
__global__ __launch_bounds__(64) void fc_clock_probe_kernel(unsigned long long *out, int samples,
                                                            unsigned long long ticksPerSample) {
    if (threadIdx.x != 0) return;
    for (int i = 0; i < samples; i++) {
        const unsigned long long r0 = wall_clock64(), c0 = clock64();
        unsigned long long r1 = r0;
        for (int poll = 0; poll < (1 << 22) && r1 - r0 < ticksPerSample; poll++) {
            __builtin_amdgcn_s_sleep(8);
            r1 = wall_clock64();
        }
        const unsigned long long c1 = clock64();
        out[2 * i] = r1 - r0;
        out[2 * i + 1] = c1 - c0;
    }
}

static const int kProbeMaxSamples = 256;

extern "C" int fc_clock_probe_begin(fc_context *ctx, int samples, int sample_us) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (samples < 1 || samples > kProbeMaxSamples || sample_us < 1 || sample_us > 100000)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_clock_probe_begin: 1..256 samples of 1..100000 us", hipSuccess);
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_clock_probe_begin: a graph is being recorded", hipSuccess);
    if (ctx->probe_samples) return fc_set_error(ctx, FC_ERR_STATE, "fc_clock_probe_begin: a probe is already running", hipSuccess);
    FC_HIP_CHECK(ctx, hipSetDevice(ctx->device));
    if (!ctx->probe_stream) FC_HIP_CHECK(ctx, hipStreamCreateWithFlags(&ctx->probe_stream, hipStreamNonBlocking));
    if (!ctx->probe_buf) FC_HIP_CHECK(ctx, hipMalloc((void **)&ctx->probe_buf, kProbeMaxSamples * 2 * sizeof(unsigned long long)));
    fc_clock_probe_kernel<<<dim3(1), dim3(64), 0, ctx->probe_stream>>>(ctx->probe_buf, samples, 100ull * sample_us);
    FC_LAUNCH_CHECK(ctx, "fc_clock_probe_kernel");
    ctx->probe_samples = samples;
    return FC_OK;
}

extern "C" int fc_clock_probe_end(fc_context *ctx, double *mhz, int capacity, int *n_samples) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!mhz || capacity < 1 || !n_samples) return fc_set_error(ctx, FC_ERR_INVALID, "fc_clock_probe_end: null or empty output", hipSuccess);
    if (!ctx->probe_samples) return fc_set_error(ctx, FC_ERR_STATE, "fc_clock_probe_end: no probe is running", hipSuccess);
    const int n = ctx->probe_samples;
    ctx->probe_samples = 0;
    FC_HIP_CHECK(ctx, hipStreamSynchronize(ctx->probe_stream));
    unsigned long long host[kProbeMaxSamples * 2];
    FC_HIP_CHECK(ctx, hipMemcpy(host, ctx->probe_buf, (size_t)n * 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    *n_samples = n;
    for (int i = 0; i < n && i < capacity; i++)
        mhz[i] = host[2 * i] ? (double)host[2 * i + 1] * 100.0 / (double)host[2 * i] : 0.0;     // ticks of 10 ns
    return FC_OK;
}

extern "C" int fc_get_device_info(fc_context *ctx, fc_device_info *info) {
    if (!fc_ctx_ok(ctx) || !info) return FC_ERR_INVALID;
    memset(info, 0, sizeof *info);
    snprintf(info->name, sizeof info->name, "%s", ctx->props.name);
    snprintf(info->arch, sizeof info->arch, "%s", ctx->props.gcnArchName);
    info->compute_units = ctx->props.multiProcessorCount;
    info->clock_mhz = ctx->props.clockRate / 1000;
    info->mem_clock_mhz = ctx->props.memoryClockRate / 1000;
    info->mem_bus_bits = ctx->props.memoryBusWidth;
    info->total_mem = ctx->props.totalGlobalMem;
    info->lds_per_block = (int)ctx->props.sharedMemPerBlock;
    return FC_OK;
}

extern "C" const char *fc_last_error(fc_context *ctx) {
    if (!fc_ctx_ok(ctx)) return "invalid context";
    return ctx->last_error.c_str();
}

extern "C" int fc_sync(fc_context *ctx) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_sync: not while a graph is recorded", hipSuccess);
    FC_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return FC_OK;
}

// ---------------------------------------------------------------- arena

static const size_t kPoolAlign = 256;

extern "C" int fc_pool_create(fc_context *ctx, size_t bytes, fc_pool **out) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!out || bytes == 0) return fc_set_error(ctx, FC_ERR_INVALID, "fc_pool_create: zero size or null out", hipSuccess);
    *out = nullptr;
    fc_pool *p = new (std::nothrow) fc_pool();
    if (!p) return FC_ERR_OOM;
    void *base = nullptr;
    hipError_t e = hipMalloc(&base, bytes);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        delete p;
        return fc_set_error(ctx, FC_ERR_OOM, "fc_pool_create: hipMalloc", e);
    }
    p->magic = FC_POOL_MAGIC;
    p->ctx = ctx;
    p->base = (char *)base;
    p->capacity = bytes;
    p->used = p->peak = 0;
    *out = p;
    return FC_OK;
}

extern "C" int fc_pool_destroy(fc_pool *pool) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    fc_context *ctx = pool->ctx;
    if (fc_ctx_ok(ctx)) (void)hipStreamSynchronize(ctx->stream);
    hipError_t e = hipFree(pool->base);
    pool->magic = 0;
    delete pool;
    if (e != hipSuccess) return fc_set_error(ctx, FC_ERR_HIP, "fc_pool_destroy: hipFree", e);
    return FC_OK;
}

extern "C" int fc_pool_alloc(fc_pool *pool, size_t bytes, void **dev_ptr) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    if (!dev_ptr) return FC_ERR_INVALID;
    *dev_ptr = nullptr;
    if (bytes == 0) return fc_set_error(pool->ctx, FC_ERR_INVALID, "fc_pool_alloc: zero bytes", hipSuccess);
    const size_t start = (pool->used + kPoolAlign - 1) / kPoolAlign * kPoolAlign;
    if (start > pool->capacity || bytes > pool->capacity - start) {
        char msg[160];
        snprintf(msg, sizeof msg, "fc_pool_alloc: %zu bytes requested, %zu of %zu in use", bytes, pool->used,
                 pool->capacity);
        return fc_set_error(pool->ctx, FC_ERR_OOM, msg, hipSuccess);
    }
    *dev_ptr = pool->base + start;
    pool->used = start + bytes;
    if (pool->used > pool->peak) pool->peak = pool->used;
    return FC_OK;
}

extern "C" int fc_pool_reset(fc_pool *pool) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    pool->used = 0;
    return FC_OK;
}

extern "C" int fc_pool_mark(fc_pool *pool, size_t *mark) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    if (!mark) return FC_ERR_INVALID;
    *mark = pool->used;
    return FC_OK;
}

extern "C" int fc_pool_release(fc_pool *pool, size_t mark) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    if (mark > pool->used) return fc_set_error(pool->ctx, FC_ERR_INVALID, "fc_pool_release: mark above current offset", hipSuccess);
    pool->used = mark;
    return FC_OK;
}

extern "C" int fc_pool_stats(fc_pool *pool, size_t *capacity, size_t *used, size_t *peak) {
    if (!pool || pool->magic != FC_POOL_MAGIC) return FC_ERR_STATE;
    if (capacity) *capacity = pool->capacity;
    if (used) *used = pool->used;
    if (peak) *peak = pool->peak;
    return FC_OK;
}

// --------------------------------------------------------------- copies

extern "C" int fc_upload(fc_context *ctx, void *dst_dev, const void *src_host, size_t bytes) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!dst_dev || !src_host) return fc_set_error(ctx, FC_ERR_INVALID, "fc_upload: null pointer", hipSuccess);
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_upload: not while a graph is recorded", hipSuccess);
    if (bytes == 0) return FC_OK;
    FC_HIP_CHECK(ctx, hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, ctx->stream));
    FC_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return FC_OK;
}

extern "C" int fc_download(fc_context *ctx, void *dst_host, const void *src_dev, size_t bytes) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!dst_host || !src_dev) return fc_set_error(ctx, FC_ERR_INVALID, "fc_download: null pointer", hipSuccess);
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_download: not while a graph is recorded", hipSuccess);
    if (bytes == 0) return FC_OK;
    FC_HIP_CHECK(ctx, hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, ctx->stream));
    FC_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    return FC_OK;
}

__global__ void fc_fill_zero_kernel(uint32_t *dst, size_t words) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < words; i += stride) dst[i] = 0u;
}

__global__ __launch_bounds__(256) void fc_fill_zero16_kernel(uint4 *dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = make_uint4(0u, 0u, 0u, 0u);
}

// A fill kernel rather than a memset node, so that callers may record it into a
// HIP graph.
extern "C" int fc_fill_zero(fc_context *ctx, void *dst_dev, size_t bytes) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!dst_dev || (bytes & 3) || ((uintptr_t)dst_dev & 3))
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_fill_zero: pointer and size must be 4-byte multiples", hipSuccess);
    if (bytes == 0) return FC_OK;
    if (((uintptr_t)dst_dev & 15) == 0 && (bytes & 15) == 0 && bytes / 16 / 256 < (1ull << 31)) {
        // 16 bytes per lane, one store per thread, as the copy kernel
        const size_t n = bytes / 16;
        fc_fill_zero16_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, ctx->stream>>>((uint4 *)dst_dev, n);
        FC_LAUNCH_CHECK(ctx, "fc_fill_zero16_kernel");
        return FC_OK;
    }
    const size_t words = bytes / 4;
    size_t blocks = (words + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    fc_fill_zero_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((uint32_t *)dst_dev, words);
    FC_LAUNCH_CHECK(ctx, "fc_fill_zero_kernel");
    return FC_OK;
}

__global__ __launch_bounds__(256) void fc_copy_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

extern "C" int fc_device_copy(fc_context *ctx, void *dst_dev, const void *src_dev, size_t bytes) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!dst_dev || !src_dev || (bytes & 15) || (((uintptr_t)dst_dev | (uintptr_t)src_dev) & 15))
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_device_copy: pointers and size must be 16-byte multiples", hipSuccess);
    if (bytes == 0) return FC_OK;
    const size_t n = bytes / 16, blocks = (n + 255) / 256;
    if (blocks >= (1ull << 31)) return fc_set_error(ctx, FC_ERR_UNSUPPORTED, "fc_device_copy: more than 512 GiB", hipSuccess);
    fc_copy_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>((const uint4 *)src_dev, (uint4 *)dst_dev, n);
    FC_LAUNCH_CHECK(ctx, "fc_copy_kernel");
    return FC_OK;
}

__global__ __launch_bounds__(256) void fc_maxpool2x2_kernel(const float *__restrict__ x, float *__restrict__ y, long planes,
                                                            int H, int W, int OH, int OW) {
    const long total = planes * OH * OW;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long)gridDim.x * 256) {
        const long pl = i / ((long)OH * OW);
        const int r = (int)(i - pl * OH * OW), oh = r / OW, ow = r - oh * OW;
        const float *src = x + (pl * H + 2 * oh) * W + 2 * ow;
        y[i] = fmaxf(fmaxf(src[0], src[1]), fmaxf(src[W], src[W + 1]));
    }
}

extern "C" int fc_maxpool2x2(fc_context *ctx, const float *x_dev, float *y_dev, int N, int C, int H, int W) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!x_dev || !y_dev || N <= 0 || C <= 0 || H < 2 || W < 2)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_maxpool2x2: bad argument", hipSuccess);
    const int OH = H / 2, OW = W / 2;
    const long total = (long)N * C * OH * OW;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    fc_maxpool2x2_kernel<<<dim3((unsigned)blocks), dim3(256), 0, ctx->stream>>>(x_dev, y_dev, (long)N * C, H, W, OH, OW);
    FC_LAUNCH_CHECK(ctx, "fc_maxpool2x2_kernel");
    return FC_OK;
}

// ---------------------------------------------------------------- graphs

// A sequence of launches recorded once and replayed with one call: for layer stacks whose
// kernels are so short that launching them one by one is what takes the time.
extern "C" int fc_graph_begin(fc_context *ctx) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_graph_begin: already recording", hipSuccess);
    if (ctx->timing_mask) return fc_set_error(ctx, FC_ERR_STATE, "fc_graph_begin: switch stage timing off first", hipSuccess);
    FC_HIP_CHECK(ctx, hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return FC_OK;
}

extern "C" int fc_graph_end(fc_context *ctx, fc_graph **out) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_graph_end: not recording", hipSuccess);
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess || !graph) return fc_set_error(ctx, FC_ERR_HIP, "hipStreamEndCapture", e);
    if (!out) {
        (void)hipGraphDestroy(graph);
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_graph_end: null output", hipSuccess);
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return fc_set_error(ctx, FC_ERR_HIP, "hipGraphInstantiate", e);
    }
    fc_graph *g = new (std::nothrow) fc_graph();
    if (!g) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return fc_set_error(ctx, FC_ERR_OOM, "fc_graph_end", hipSuccess);
    }
    g->magic = FC_GRAPH_MAGIC; g->ctx = ctx; g->graph = graph; g->exec = exec;
    *out = g;
    return FC_OK;
}

extern "C" int fc_graph_launch(fc_context *ctx, fc_graph *g) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (!g || g->magic != FC_GRAPH_MAGIC || g->ctx != ctx)
        return fc_set_error(ctx, FC_ERR_INVALID, "fc_graph_launch: not a graph of this context", hipSuccess);
    if (ctx->capturing) return fc_set_error(ctx, FC_ERR_STATE, "fc_graph_launch: recording", hipSuccess);
    FC_HIP_CHECK(ctx, hipGraphLaunch(g->exec, ctx->stream));
    return FC_OK;
}

extern "C" int fc_graph_destroy(fc_graph *g) {
    if (!g || g->magic != FC_GRAPH_MAGIC) return FC_ERR_INVALID;
    if (fc_ctx_ok(g->ctx)) (void)hipStreamSynchronize(g->ctx->stream);
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    g->magic = 0;
    delete g;
    return FC_OK;
}

// --------------------------------------------------------------- timing

static int fc_timing_fold(fc_context *ctx) {
    if (ctx->pending.empty()) return FC_OK;
    FC_HIP_CHECK(ctx, hipStreamSynchronize(ctx->stream));
    for (auto &p : ctx->pending) {
        float ms = 0.f;
        FC_HIP_CHECK(ctx, hipEventElapsedTime(&ms, p.start, p.stop));
        ctx->stage_ms[p.stage] += ms;
        ctx->stage_launches[p.stage] += 1;
        ctx->free_events.push_back(p.start);
        ctx->free_events.push_back(p.stop);
    }
    ctx->pending.clear();
    return FC_OK;
}

static hipEvent_t fc_take_event(fc_context *ctx) {
    if (!ctx->free_events.empty()) {
        hipEvent_t ev = ctx->free_events.back();
        ctx->free_events.pop_back();
        return ev;
    }
    hipEvent_t ev = nullptr;
    if (hipEventCreate(&ev) != hipSuccess) return nullptr;
    return ev;
}

fc_stage_scope::fc_stage_scope(fc_context *c, int stage) : ctx(c), stop(nullptr), active(false) {
    if (stage < 0 || !(c->timing_mask & (1u << stage))) return;      // stage -1: never bracketed
    if (c->pending.size() >= 8192) (void)fc_timing_fold(c);
    hipEvent_t start = fc_take_event(c);
    stop = fc_take_event(c);
    if (!start || !stop) return;
    (void)hipEventRecord(start, c->stream);
    c->pending.push_back({stage, start, stop});
    active = true;
}

fc_stage_scope::~fc_stage_scope() {
    if (active) (void)hipEventRecord(stop, ctx->stream);
}

extern "C" int fc_timing_enable(fc_context *ctx, int stage_mask) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (ctx->capturing && stage_mask)
        return fc_set_error(ctx, FC_ERR_STATE, "fc_timing_enable: not while a graph is recorded", hipSuccess);
    if (!stage_mask) {
        const int rc = fc_timing_fold(ctx);
        if (rc) return rc;
    }
    ctx->timing_mask = (unsigned)stage_mask & ((1u << FC_STAGE_COUNT) - 1);
    return FC_OK;
}

extern "C" int fc_timing_reset(fc_context *ctx) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    const int rc = fc_timing_fold(ctx);
    if (rc) return rc;
    memset(ctx->stage_ms, 0, sizeof ctx->stage_ms);
    memset(ctx->stage_launches, 0, sizeof ctx->stage_launches);
    return FC_OK;
}

extern "C" int fc_stage_time_ms(fc_context *ctx, int stage, double *total_ms, long *launches) {
    if (!fc_ctx_ok(ctx)) return FC_ERR_STATE;
    if (stage < 0 || stage >= FC_STAGE_COUNT) return fc_set_error(ctx, FC_ERR_INVALID, "fc_stage_time_ms: stage", hipSuccess);
    const int rc = fc_timing_fold(ctx);
    if (rc) return rc;
    if (total_ms) *total_ms = ctx->stage_ms[stage];
    if (launches) *launches = ctx->stage_launches[stage];
    return FC_OK;
}
