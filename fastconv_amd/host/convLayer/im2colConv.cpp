#include "im2colConv.h"

#include "../utility/tuning_log.h"

using fastconv::Device;

ConvIm2colLayer::ConvIm2colLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih,
                                 size_t iw, size_t oc, size_t kh, size_t kw, size_t sh, size_t sw, size_t pad_left,
                                 size_t pad_right, size_t pad_top, size_t pad_bottom, size_t g, bool bias, size_t nt,
                                 size_t iter, size_t n, int tile_config)
    : ConvLayer(input, kernel, biasw, output_ref, ic, ih, iw, oc, kh, kw, sh, sw, pad_left, pad_right, pad_top,
                pad_bottom, g, bias, nt, iter, n) {
    this->M = (int)output_channels;
    this->N = (long)batch * output_height * output_width;
    this->K = (int)(input_channels * kernel_height * kernel_width);
    packed_kernel = NULL;
    gather_table = NULL;
    workspace = NULL;
    channel_bias = NULL;
    relu = false;
    if (bias) fprintf(stderr, "Warning: the per-element bias tensor is ignored by the im2col layer (use SetChannelBias)\n");
    config_best = tile_config;
    if (config_best < 0 || config_best >= fc_igemm_num_configs()) {
        const fc_conv_shape s = Shape();
        config_best = fc_igemm_default_config(&s);
        if (config_best < 0) config_best = 0;
    }
    config = config_best;
}

ConvIm2colLayer::~ConvIm2colLayer() { dev.Release(); }

fc_conv_shape ConvIm2colLayer::Shape() const {
    fc_conv_shape s;
    s.N = (int)batch; s.C = (int)input_channels; s.H = (int)input_height; s.W = (int)input_width;
    s.K = (int)output_channels; s.kh = (int)kernel_height; s.kw = (int)kernel_width;
    s.sh = (int)stride_height; s.sw = (int)stride_width;
    s.pt = (int)padding_top; s.pb = (int)padding_bottom; s.pl = (int)padding_left; s.pr = (int)padding_right;
    return s;
}

void ConvIm2colLayer::SetChannelBias(const float *bias_k, bool relu_) {
    channel_bias = bias_k;
    relu = relu_;
}

// Plans one tile shape and re-lays the filter for it (the one-time counterpart
// of the reference's per-call pack_a, im2col/gemm_pack.cpp:192-260).
void ConvIm2colLayer::AllocateFor(int cfg) {
    Device &d = Device::Get();
    const fc_conv_shape s = Shape();
    const int rc = fc_igemm_make_plan(&s, cfg, &plan);
    if (rc != FC_OK) {
        fprintf(stderr, "Error: no implicit-GEMM plan for this layer: %s\n", fc_status_string(rc));
        exit(EXIT_FAILURE);
    }
    config = cfg;
    packed_kernel = (float *)d.Alloc(plan.Wp_bytes, "packed kernel");
    gather_table = (int32_t *)d.Alloc(plan.table_bytes, "gather table");
    workspace = plan.ws_bytes ? (float *)d.Alloc(plan.ws_bytes, "split-reduction workspace") : NULL;
    d.Check(fc_igemm_pack_filter(d.ctx(), &plan, dev.kernel, packed_kernel, gather_table), "fc_igemm_pack_filter");
}

void ConvIm2colLayer::RunOnce() {
    Device &d = Device::Get();
    d.Check(fc_conv_implicit_gemm(d.ctx(), &plan, dev.input, packed_kernel, gather_table, dev.bias, relu ? 1 : 0,
                                  workspace, dev.output),
            "fc_conv_implicit_gemm");
}

int ConvIm2colLayer::Init() {
    printf("Algorithm: im2col\n");
    const size_t in_elems = batch * input_channels * input_height * input_width;
    dev.Acquire(input_data, in_elems, kernel_data, (size_t)M * K, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);
    AllocateFor(config_best);
    fc_gemm_config c;
    fc_igemm_get_config(config, &c);
    printf("Testing M=%d N=%ld K=%d batch=%zu tile %dx%dx%d (cfg %d) reduction split %d over workgroups, %d over wavefronts\n",
           M, N, K, batch, c.bm, c.bn, c.bk, config, plan.split_k, c.waves_k);
    return 1;
}

int ConvIm2colLayer::Forward() {
    Device &d = Device::Get();
    if (!packed_kernel) {
        fprintf(stderr, "Error: Forward() before Init()\n");
        exit(EXIT_FAILURE);
    }
    RunOnce();
    d.Check(fc_sync(d.ctx()), "fc_sync");
    Timer total;
    total.startBench();
    for (size_t i = 0; i < iterations; i++) RunOnce();
    d.Check(fc_sync(d.ctx()), "fc_sync");
    total.accumBench();

    d.Check(fc_timing_enable(d.ctx(), FC_TIMING_ALL), "fc_timing_enable");
    d.Check(fc_timing_reset(d.ctx()), "fc_timing_reset");
    for (size_t i = 0; i < iterations; i++) RunOnce();
    double ms = 0;
    long cnt = 0;
    d.Check(fc_stage_time_ms(d.ctx(), FC_STAGE_IMPLICIT_GEMM, &ms, &cnt), "fc_stage_time_ms");
    d.Check(fc_timing_enable(d.ctx(), 0), "fc_timing_enable");
    gemm_ms = ms / iterations;
    // the column matrix is built inside the GEMM kernel: there is no separate transform stage
    LOGD("%s %lfms\n", "Im2colTran time:", 0.0);
    LOGD("%s %lfms\n", "Gemm time:", gemm_ms);
    total.printBench("Total time:", (int)iterations);
    last_total_ms = total.accumulated() / iterations;

    dev.Download(output_data, output_elements());
    if (output_ref != NULL) diff(output_ref, output_data, (int)output_elements());
    return 1;
}

int ConvIm2colLayer::Tuning() {
    Device &d = Device::Get();
    const fc_conv_shape s = Shape();
    TuningKey key = {"im2col", s.N, s.C, s.H, s.W, s.K, s.kh, s.kw, s.sh, s.sw, s.pt, s.pb, s.pl, s.pr};
    TuningEntry hit;
    if (tuning_log_lookup(key, &hit) && hit.config >= 0 && hit.config < fc_igemm_num_configs()) {
        printf("log entry exists.\n");
        config_best = hit.config;
        return 1;
    }
    printf("log entry doesn't exist.\n");
    const size_t in_elems = batch * input_channels * input_height * input_width;
    dev.Acquire(input_data, in_elems, kernel_data, (size_t)M * K, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);
    double best_ms = 1e100;
    for (int cfg = 0; cfg < fc_igemm_num_configs(); cfg++) {
        fc_igemm_plan probe;
        if (fc_igemm_make_plan(&s, cfg, &probe) != FC_OK) continue;      // a tile shape that cannot run this layer
        const size_t mark = d.Mark();
        AllocateFor(cfg);
        RunOnce();
        d.Check(fc_sync(d.ctx()), "fc_sync");
        Timer t;
        t.startBench();
        for (size_t i = 0; i < iterations; i++) RunOnce();
        d.Check(fc_sync(d.ctx()), "fc_sync");
        const double ms = t.endBench((double)iterations);
        fc_gemm_config c;
        fc_igemm_get_config(cfg, &c);
        float dis = 0.f;
        if (output_ref != NULL) {
            dev.Download(output_data, output_elements());
            dis = diff(output_ref, output_data, (int)output_elements());
        }
        printf("M=%d N=%ld K=%d tile %dx%dx%d waves %dx%dx%d cfg=%d time=%.3f, diff=%.3f\n", M, N, K, c.bm, c.bn, c.bk,
               c.waves_m, c.waves_n, c.waves_k, cfg, ms, dis);
        if (ms < best_ms) {
            best_ms = ms;
            config_best = cfg;
        }
        d.Release(mark);
        packed_kernel = NULL;
        gather_table = NULL;
    }
    dev.Release();
    TuningEntry e = {config_best, 0, best_ms};
    tuning_log_append(key, e);
    printf("Best Config: (M=%d N=%ld K=%d) cfg=%d time=%.3f\n", M, N, K, config_best, best_ms);
    return 1;
}
