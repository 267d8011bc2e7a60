#include "winoF63Conv.h"

#include "../utility/tuning_log.h"
#include "winoF63ConvZC.h"

using fastconv::Device;

static const size_t kCacheBudget = (size_t)8 << 30;   // V of one block of images; by default the whole batch is one block

ConvWinoF63Layer::ConvWinoF63Layer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih,
                                   size_t iw, size_t oc, size_t kh, size_t kw, size_t sh, size_t sw, size_t pad_left,
                                   size_t pad_right, size_t pad_top, size_t pad_bottom, size_t g, bool bias, size_t nt,
                                   size_t iter, size_t n)
    : ConvLayer(input, kernel, biasw, output_ref, ic, ih, iw, oc, kh, kw, sh, sw, pad_left, pad_right, pad_top,
                pad_bottom, g, bias, nt, iter, n) {
    inputBuf = gemmBuf = kernelBuf = NULL;
    onePass = false;
    channel_bias = NULL;
    relu = false;
    hasTail = false;
    if (kh != 3 || kw != 3 || sh != 1 || sw != 1) {
        fprintf(stderr, "Error: Winograd F(6x6,3x3) needs a 3x3 kernel and stride 1\n");
        exit(EXIT_FAILURE);
    }
    if (bias) fprintf(stderr, "Warning: the per-element bias tensor is ignored by the Winograd layer (use SetChannelBias)\n");
    const size_t tileN = ((output_height + 5) / 6) * ((output_width + 5) / 6);
    imgBlock_best = DefaultImagesPerBlock(oc, ic, tileN, n, kCacheBudget);
    gemmConfig_best = ConvWinoF63ZCLayer::DefaultConfig(oc, ic, ih, iw, pad_top, imgBlock_best);
    const fc_conv_shape whole = Shape((int)n);
    if (fc_wino_prefer_onepass(&whole)) imgBlock_best = 0;      // 0: the single-kernel engine, whole batch
    enableOffKernel = enableOffKernel_best = 0;      // online, as the driver's -ts default
    tileBlock = ocBlock = icBlock = ocRegBlock = tileRegBlock = imgBlock = 0;
}

ConvWinoF63Layer::~ConvWinoF63Layer() { dev.Release(); }

int ConvWinoF63Layer::DefaultImagesPerBlock(size_t K, size_t C, size_t tileN, size_t N, size_t budget) {
    (void)K;
    const size_t per_image = 64 * 4 * C * tileN;
    size_t b = budget / (per_image ? per_image : 1);
    if (b < 1) b = 1;
    if (b > N) b = N;
    return (int)b;
}

fc_conv_shape ConvWinoF63Layer::Shape(int n) const {
    fc_conv_shape s;
    s.N = n; s.C = (int)input_channels; s.H = (int)input_height; s.W = (int)input_width;
    s.K = (int)output_channels; s.kh = 3; s.kw = 3; s.sh = 1; s.sw = 1;
    s.pt = (int)padding_top; s.pb = (int)padding_bottom; s.pl = (int)padding_left; s.pr = (int)padding_right;
    return s;
}

void ConvWinoF63Layer::SetChannelBias(const float *bias_k, bool relu_) {
    channel_bias = bias_k;
    relu = relu_;
}

void ConvWinoF63Layer::SetConfig(int gemm_config, int images_per_block) {
    gemmConfig_best = gemm_config;
    imgBlock_best = images_per_block < 0 ? 1 : (images_per_block > (int)batch ? (int)batch : images_per_block);
}

void ConvWinoF63Layer::AllocateFor(int config, int images_per_block) {
    Device &d = Device::Get();
    onePass = images_per_block == 0;
    if (onePass) {
        // input transform, products and output transform in one kernel: the block-local scratch of
        // the reference is LDS and registers, and there is no reason left to cut the batch
        imgBlock = (int)batch;
        hasTail = false;
        fc_conv_shape whole = Shape(imgBlock);
        const int orc = fc_wino_make_onepass_plan(&whole, &plan);
        if (orc != FC_OK) {
            fprintf(stderr, "Error: no single-kernel Winograd plan for this layer: %s\n", fc_status_string(orc));
            exit(EXIT_FAILURE);
        }
        ocBlock = 64; icBlock = 4; ocRegBlock = 4; tileRegBlock = 1;
        tileBlock = 16;
        inputBuf = gemmBuf = NULL;
        kernelBuf = (float *)d.Alloc(plan.U_bytes, "kernelBuf");
        if (enableOffKernel)
            d.Check(fc_wino_onepass_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_onepass_filter_transform");
        return;
    }
    imgBlock = images_per_block;
    fc_conv_shape s = Shape(imgBlock);
    int rc = fc_wino_make_plan(&s, config, &plan);
    const int tail = (int)(batch % imgBlock);
    hasTail = tail != 0;
    if (rc == FC_OK && hasTail) {
        s = Shape(tail);
        rc = fc_wino_make_plan(&s, config, &tailPlan);
    }
    if (rc != FC_OK) {
        fprintf(stderr, "Error: no Winograd plan for this layer: %s\n", fc_status_string(rc));
        exit(EXIT_FAILURE);
    }
    fc_gemm_config c;
    fc_wino_gemm_get_config(config, &c);
    ocBlock = c.bm; icBlock = c.bk; ocRegBlock = c.waves_m; tileRegBlock = c.waves_n;
    tileBlock = (int)plan.T;
    inputBuf = (float *)d.Alloc(plan.V_bytes, "inputBuf");
    gemmBuf = NULL;      // the per-frequency products live in registers and LDS only
    kernelBuf = (float *)d.Alloc(plan.U_bytes, "kernelBuf");
    // U does not depend on the batch: one transform serves the full and the tail plan
    if (enableOffKernel)
        d.Check(fc_wino_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_filter_transform");
}

// split_stages: an online filter transform gets a launch of its own (otherwise it rides in the input
// transform's launch), so that its time can be listed by itself.
void ConvWinoF63Layer::RunOnce(bool split_stages) {
    Device &d = Device::Get();
    const size_t in_img = input_channels * input_height * input_width;
    const size_t out_img = output_channels * output_height * output_width;
    if (onePass) {
        d.Check(fc_wino_forward_onepass(d.ctx(), &plan, dev.input, dev.kernel, dev.bias, relu ? 1 : 0, enableOffKernel,
                                        kernelBuf, dev.output),
                "fc_wino_forward_onepass");
        return;
    }
    const bool split = split_stages && !enableOffKernel;
    if (split) d.Check(fc_wino_filter_transform(d.ctx(), &plan, dev.kernel, kernelBuf), "fc_wino_filter_transform");
    for (size_t n0 = 0; n0 < batch; n0 += imgBlock) {
        const fc_wino_plan *p = (n0 + imgBlock <= batch) ? &plan : &tailPlan;
        // online: the filter is transformed with the first block of every pass
        d.Check(fc_wino_forward_fused(d.ctx(), p, dev.input + n0 * in_img, dev.kernel, dev.bias, relu ? 1 : 0,
                                      (enableOffKernel || split || n0 > 0) ? 1 : 0, kernelBuf, inputBuf, dev.output + n0 * out_img),
                "fc_wino_forward_fused");
    }
}

int ConvWinoF63Layer::Tuning() {
    Device &d = Device::Get();
    const fc_conv_shape s = Shape((int)batch);
    TuningKey key = {"winograd_blocked", s.N, s.C, s.H, s.W, s.K, 3, 3, 1, 1, s.pt, s.pb, s.pl, s.pr};
    TuningEntry hit;
    if (tuning_log_lookup(key, &hit) && hit.config >= 0 && hit.config < fc_wino_gemm_num_configs()) {
        printf("log entry exists.\n");
        // option = 2 * images per block + offline flag
        SetConfig(hit.config, hit.option / 2);
        enableOffKernel_best = hit.option % 2;
        printf("Best Config: (%zu %zu %zu) cfg=%d imgb=%d eoffK%d time=%.3f\n", input_channels, output_channels, input_width,
               gemmConfig_best, imgBlock_best, enableOffKernel_best, hit.ms);
        return -1;
    }
    printf("log entry doesn't exist.\n");
    const size_t in_elems = batch * input_channels * input_height * input_width;
    dev.Acquire(input_data, in_elems, kernel_data, output_channels * input_channels * 9, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);

    double minTimeusage = 1e100;
    for (int cfg = 0; cfg < fc_wino_gemm_num_configs(); cfg++) {
        // images per block 0 is the single-kernel engine (no tile shape: tried once)
        for (int ib = (cfg == 0 ? 0 : 1); ib <= (int)batch; ib = ib ? ib * 2 : 1) {
            fc_wino_plan probe;
            fc_conv_shape ps = Shape(ib ? ib : (int)batch);
            if (ib == 0) {
                if (fc_wino_make_onepass_plan(&ps, &probe) != FC_OK) continue;
            } else if (fc_wino_make_plan(&ps, cfg, &probe) != FC_OK) continue;
            size_t cap, used, peak;
            fc_pool_stats(d.pool(), &cap, &used, &peak);
            if (probe.U_bytes + probe.V_bytes + 4096 > cap - used) continue;
          for (enableOffKernel = 1; enableOffKernel >= 0; enableOffKernel--) {
            const size_t mark = d.Mark();
            AllocateFor(cfg, ib);
            RunOnce();
            d.Check(fc_sync(d.ctx()), "fc_sync");
            timespec start, stop;
            clock_gettime(CLOCK_MONOTONIC, &start);
            for (size_t i = 0; i < iterations; i++) RunOnce();
            d.Check(fc_sync(d.ctx()), "fc_sync");
            clock_gettime(CLOCK_MONOTONIC, &stop);
            const double elapsedTime =
                ((stop.tv_sec - start.tv_sec) * 1000.0 + (stop.tv_nsec - start.tv_nsec) / 1000000.0) / iterations;
            float dis = 0.f;
            if (output_ref != NULL) {
                dev.Download(output_data, output_elements());
                dis = diff(output_ref, output_data, (int)output_elements());
            }
            printf("ocb=%d tb=%d icb=%d ocr%d tbr%d cfg=%d imgb=%d eoffK%d time=%.3f, diff=%.3f\n", ocBlock, tileBlock,
                   icBlock, ocRegBlock, tileRegBlock, cfg, ib, enableOffKernel, elapsedTime, dis);
            if (minTimeusage > elapsedTime) {
                gemmConfig_best = cfg;
                imgBlock_best = ib;
                enableOffKernel_best = enableOffKernel;
                minTimeusage = elapsedTime;
            }
            d.Release(mark);
            inputBuf = gemmBuf = kernelBuf = NULL;
          }
        }
    }
    dev.Release();
    TuningEntry e = {gemmConfig_best, 2 * imgBlock_best + enableOffKernel_best, minTimeusage};
    tuning_log_append(key, e);
    printf("Best Config: (%zu %zu %zu) cfg=%d imgb=%d eoffK%d time=%.3f\n", input_channels, output_channels, input_width,
           gemmConfig_best, imgBlock_best, enableOffKernel_best, minTimeusage);
    return -1;
}

int ConvWinoF63Layer::Init() {
    const size_t in_elems = batch * input_channels * input_height * input_width;
    dev.Acquire(input_data, in_elems, kernel_data, output_channels * input_channels * 9, output_elements());
    if (channel_bias) dev.SetBias(channel_bias, output_channels);
    enableOffKernel = enableOffKernel_best;
    AllocateFor(gemmConfig_best, imgBlock_best);
    printf("Algorithm: winograd F63 (blocked%s)\n", onePass ? ", single kernel" : "");
    if (enableOffKernel) printf("offline kernel transform.\n");
    printf("enableoffkernel = %d\n", enableOffKernel);
    printf("Testing ic=%zu oc=%zu width=%zu batch=%zu tileBlock=%d (%d images) ocBlock=%d icBlock=%d\n", input_channels,
           output_channels, input_width, batch, tileBlock, imgBlock, ocBlock, icBlock);
    printf("kernelBuf %zu KB\n", plan.U_bytes / 1024);
    printf("gemmBuf   %d KB (LDS per workgroup, no device buffer)\n", onePass ? 144 : 128);
    printf("inputBuf  %zu KB\n", plan.V_bytes / 1024);
    return -1;
}

int ConvWinoF63Layer::Forward() {
    Device &d = Device::Get();
    if (!kernelBuf) {
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
    for (size_t i = 0; i < iterations; i++) RunOnce(true);
    // the GEMM and the output transform are one kernel here: its time is listed as TensorGEMM
    // (with the single-kernel engine that one kernel also holds the input transform)
    const int stages[4] = {FC_STAGE_INPUT_TRAN, FC_STAGE_KERNEL_TRAN, onePass ? FC_STAGE_ONEPASS : FC_STAGE_FUSED_GEMM_OUT,
                           FC_STAGE_OUTPUT_TRAN};
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
