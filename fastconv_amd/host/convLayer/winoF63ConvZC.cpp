#include "winoF63ConvZC.h"

#include "../utility/tuning_log.h"

using fastconv::Device;

ConvWinoF63ZCLayer::ConvWinoF63ZCLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic,
                                       size_t ih, size_t iw, size_t oc, size_t kh, size_t kw, size_t sh, size_t sw,
                                       size_t pad_left, size_t pad_right, size_t pad_top, size_t pad_bottom, size_t g,
                                       bool bias, size_t nt, size_t iter, size_t n)
    : ConvLayer(input, kernel, biasw, output_ref, ic, ih, iw, oc, kh, kw, sh, sw, pad_left, pad_right, pad_top,
                pad_bottom, g, bias, nt, iter, n) {
    inputBuf = gemmBuf = kernelBuf = NULL;
    channel_bias = NULL;
    relu = false;
    if (kh != 3 || kw != 3 || sh != 1 || sw != 1) {
        fprintf(stderr, "Error: Winograd F(6x6,3x3) needs a 3x3 kernel and stride 1\n");
        exit(EXIT_FAILURE);
    }
    if (bias) fprintf(stderr, "Warning: the per-element bias tensor is ignored by the Winograd layer (use SetChannelBias)\n");
    gemmConfig_best = DefaultConfig(oc, ic, ih, iw, pad_top, n);
    scheduling_best = 0;
    gemmConfig = gemmConfig_best;
    enableOffKernel = scheduling = 0;
    tileBlock = ocBlock = icBlock = ocRegBlock = tileRegBlock = 0;
}

ConvWinoF63ZCLayer::~ConvWinoF63ZCLayer() { dev.Release(); }

// Tile shape used without tuning: the library's cost model.
int ConvWinoF63ZCLayer::DefaultConfig(size_t K, size_t C, size_t H, size_t W, size_t pad, size_t N) {
    fc_conv_shape s;
    s.N = (int)N; s.C = (int)C; s.H = (int)H; s.W = (int)W; s.K = (int)K;
    s.kh = s.kw = 3; s.sh = s.sw = 1; s.pt = s.pb = s.pl = s.pr = (int)pad;
    const int id = fc_wino_gemm_default_config(&s);
    return id < 0 ? 0 : id;
}

fc_conv_shape ConvWinoF63ZCLayer::Shape() const {
    fc_conv_shape s;
    s.N = (int)batch; s.C = (int)input_channels; s.H = (int)input_height; s.W = (int)input_width;
    s.K = (int)output_channels; s.kh = 3; s.kw = 3; s.sh = 1; s.sw = 1;
    s.pt = (int)padding_top; s.pb = (int)padding_bottom; s.pl = (int)padding_left; s.pr = (int)padding_right;
    return s;
}

void ConvWinoF63ZCLayer::SetChannelBias(const float *bias_k, bool relu_) {
    channel_bias = bias_k;
    relu = relu_;
}

void ConvWinoF63ZCLayer::SetConfig(int gemm_config, int offline) {
    gemmConfig_best = gemm_config;
    scheduling_best = offline ? 1 : 0;
}

// Allocates U, V, M for one tile configuration (the counterpart of the
// inputBuf/gemmBuf/kernelBuf sizing in the reference's Init and Tuning).
void ConvWinoF63ZCLayer::AllocateFor(int config) {
    Device &d = Device::Get();
    const fc_conv_shape s = Shape();
    const int rc = fc_wino_make_plan(&s, config, &plan);
    if (rc != FC_OK) {
        fprintf(stderr, "Error: no Winograd plan for this layer: %s\n", fc_status_string(rc));
        exit(EXIT_FAILURE);
    }
    fc_gemm_config c;
    fc_wino_gemm_get_config(config, &c);
    gemmConfig = config;
    ocBlock = c.bm; tileBlock = c.bn; icBlock = c.bk; ocRegBlock = c.waves_m; tileRegBlock = c.waves_n;
    inputBuf = (float *)d.Alloc(plan.V_bytes, "inputBuf");
    gemmBuf = (float *)d.Alloc(plan.M_bytes, "gemmBuf");
    kernelBuf = (float *)d.Alloc(plan.U_bytes, "kernelBuf");
}

void ConvWinoF63ZCLayer::RunOnce(bool filter_ready) {
    Device &d = Device::Get();
    d.Check(fc_wino_forward(d.ctx(), &plan, dev.input, dev.kernel, dev.bias, relu ? 1 : 0, filter_ready ? 1 : 0,
                            kernelBuf, inputBuf, gemmBuf, dev.output),
            "fc_wino_forward");
}

// The four stages as four launches (RunOnce puts the two transforms into one): used for the
// per-stage times, which the reference prints one by one.
void ConvWinoF63ZCLayer::RunStages(bool filter_ready) {
    Device &d = Device::Get();
    // few tiles and an online filter: the products are made straight from the 3x3 taps (as RunOnce does)
    const bool raw = !filter_ready && fc_wino_prefer_raw_filter_gemm(&plan);
    if (!filter_ready && !raw)
        d.Check(fc_wino_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_filter_transform");
    d.Check(fc_wino_input_transform(d.ctx(), &plan, dev.input, inputBuf), "fc_wino_input_transform");
    if (raw) d.Check(fc_wino_gemm_raw_filter(d.ctx(), &plan, dev.kernel, inputBuf, gemmBuf, 0, 0), "fc_wino_gemm_raw_filter");
    else d.Check(fc_wino_gemm(d.ctx(), &plan, kernelBuf, inputBuf, gemmBuf), "fc_wino_gemm");
    d.Check(fc_wino_output_transform(d.ctx(), &plan, gemmBuf, dev.bias, relu ? 1 : 0, dev.output), "fc_wino_output_transform");
}

int ConvWinoF63ZCLayer::Tuning() {
    Device &d = Device::Get();
    const fc_conv_shape s = Shape();
    TuningKey key = {"winograd_zc", s.N, s.C, s.H, s.W, s.K, 3, 3, 1, 1, s.pt, s.pb, s.pl, s.pr};
    TuningEntry hit;
    if (tuning_log_lookup(key, &hit) && hit.config >= 0 && hit.config < fc_wino_gemm_num_configs()) {
        printf("log entry exists.\n");
        gemmConfig_best = hit.config;
        scheduling_best = hit.option;
        printf("Best Config: (%zu %zu %zu) cfg=%d eoffK%d time=%.3f\n", input_channels, output_channels, input_width,
               gemmConfig_best, scheduling_best % 2, hit.ms);
        return -1;
    }
    printf("log entry doesn't exist.\n");

    const size_t in_elems = batch * input_channels * input_height * input_width;
    const size_t k_elems = output_channels * input_channels * 9;
    dev.Acquire(input_data, in_elems, kernel_data, k_elems, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);

    double minTimeusage = 1e100;
    const int warmup = 1;
    for (int cfg = 0; cfg < fc_wino_gemm_num_configs(); cfg++) {
        fc_wino_plan probe;
        if (fc_wino_make_plan(&s, cfg, &probe) != FC_OK) continue;
        size_t cap, used, peak;
        fc_pool_stats(d.pool(), &cap, &used, &peak);
        if (probe.U_bytes + probe.V_bytes + probe.M_bytes + 4096 > cap - used) {
            printf("cfg=%d skipped: needs %zu MiB of scratch\n", cfg,
                   (probe.U_bytes + probe.V_bytes + probe.M_bytes) >> 20);
            continue;
        }
        for (enableOffKernel = 1; enableOffKernel >= 0; enableOffKernel--) {
            const size_t mark = d.Mark();
            AllocateFor(cfg);
            if (enableOffKernel)
                d.Check(fc_wino_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_filter_transform");
            for (int i = 0; i < warmup; i++) RunOnce(enableOffKernel != 0);
            d.Check(fc_sync(d.ctx()), "fc_sync");
            timespec start, stop;
            clock_gettime(CLOCK_MONOTONIC, &start);
            for (size_t i = 0; i < iterations; i++) RunOnce(enableOffKernel != 0);
            d.Check(fc_sync(d.ctx()), "fc_sync");
            clock_gettime(CLOCK_MONOTONIC, &stop);
            const double elapsedTime =
                ((stop.tv_sec - start.tv_sec) * 1000.0 + (stop.tv_nsec - start.tv_nsec) / 1000000.0) / iterations;
            if (output_ref != NULL) {
                dev.Download(output_data, output_elements());
                const float dis = diff(output_ref, output_data, (int)output_elements());
                printf("ocb=%d tb=%d icb=%d ocr%d tbr%d cfg=%d eoffK%d time=%.3f, diff=%.3f\n", ocBlock, tileBlock, icBlock,
                       ocRegBlock, tileRegBlock, cfg, enableOffKernel, elapsedTime, dis);
            } else {
                printf("ocb=%d tb=%d icb=%d ocr%d tbr%d cfg=%d eoffK%d time=%.3f\n", ocBlock, tileBlock, icBlock,
                       ocRegBlock, tileRegBlock, cfg, enableOffKernel, elapsedTime);
            }
            if (minTimeusage > elapsedTime) {
                gemmConfig_best = cfg;
                scheduling_best = enableOffKernel;
                minTimeusage = elapsedTime;
            }
            d.Release(mark);
            inputBuf = gemmBuf = kernelBuf = NULL;
        }
    }
    dev.Release();
    TuningEntry e = {gemmConfig_best, scheduling_best, minTimeusage};
    tuning_log_append(key, e);
    printf("Best Config: (%zu %zu %zu) cfg=%d eoffK%d time=%.3f\n", input_channels, output_channels, input_width,
           gemmConfig_best, scheduling_best % 2, minTimeusage);
    return -1;
}

int ConvWinoF63ZCLayer::Init() {
    Device &d = Device::Get();
    scheduling = scheduling_best;
    enableOffKernel = scheduling % 2;

    const size_t in_elems = batch * input_channels * input_height * input_width;
    const size_t k_elems = output_channels * input_channels * 9;
    dev.Acquire(input_data, in_elems, kernel_data, k_elems, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);
    AllocateFor(gemmConfig_best);

    printf("Algorithm: winograd F63\n");
    printf("Testing ic=%zu oc=%zu width=%zu batch=%zu tileBlock=%d ocBlock=%d icBlock=%d (cfg %d) tiles=%ld\n",
           input_channels, output_channels, input_width, batch, tileBlock, ocBlock, icBlock, gemmConfig, plan.T);
    if (enableOffKernel) {
        d.Check(fc_wino_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_filter_transform");
        printf("offline kernel transform.\n");
    }
    return -1;
}

int ConvWinoF63ZCLayer::Forward() {
    Device &d = Device::Get();
    if (!inputBuf) {
        fprintf(stderr, "Error: Forward() before Init()\n");
        exit(EXIT_FAILURE);
    }
    // one untimed pass: first-launch costs are not part of a stage time
    RunOnce(enableOffKernel != 0);
    d.Check(fc_sync(d.ctx()), "fc_sync");

    // pass 1: whole-iteration wall time with the stages launched back to back
    Timer total;
    total.startBench();
    for (size_t i = 0; i < iterations; i++) RunOnce(enableOffKernel != 0);
    d.Check(fc_sync(d.ctx()), "fc_sync");
    total.accumBench();

    // pass 2: the same iterations with every stage bracketed by events
    d.Check(fc_timing_enable(d.ctx(), FC_TIMING_ALL), "fc_timing_enable");
    d.Check(fc_timing_reset(d.ctx()), "fc_timing_reset");
    for (size_t i = 0; i < iterations; i++) RunStages(enableOffKernel != 0);
    const int stages[4] = {FC_STAGE_INPUT_TRAN, FC_STAGE_KERNEL_TRAN, FC_STAGE_TENSOR_GEMM, FC_STAGE_OUTPUT_TRAN};
    const char *labels[4] = {"InputTran time:", "KernelTran time:", "TensorGEMM time:", "OutputTran time:"};
    for (int i = 0; i < 4; i++) {
        double ms = 0;
        long cnt = 0;
        d.Check(fc_stage_time_ms(d.ctx(), stages[i], &ms, &cnt), "fc_stage_time_ms");
        stage_ms[i] = ms / iterations;
        LOGD("%s %lfms\n", labels[i], stage_ms[i]);
    }
    d.Check(fc_timing_enable(d.ctx(), 0), "fc_timing_enable");
    total.printBench("Total time:", (int)iterations);
    last_total_ms = total.accumulated() / iterations;

    dev.Download(output_data, output_elements());
    if (output_ref != NULL) diff(output_ref, output_data, (int)output_elements());
    return 1;
}
