// Winograd F(6x6,3x3) layer, staged "zero copy" pipeline: four kernels over
// whole-layer buffers U, V, M in their final layouts (filter transform, input
// transform, 64 batched fp32-MFMA GEMMs, output transform fused with the NCHW
// write-back).  Interface of the reference's ConvWinoF63ZCLayer
// (convLayer/winoF63ConvZC.h:9-43): same constructor (plus batch), Tuning() ->
// Init() -> Forward().
#ifndef WINOF63CONVZC_H_
#define WINOF63CONVZC_H_

#include "../conv_layer.h"
#include "../utility/helper.h"
#include "deviceBuffers.h"
#include "fastconv_hip.h"

class ConvWinoF63ZCLayer : public ConvLayer {
   public:
    ConvWinoF63ZCLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih, size_t iw,
                       size_t oc, size_t kh = 3, size_t kw = 3, size_t sh = 1, size_t sw = 1, size_t pad_left = 1,
                       size_t pad_right = 1, size_t pad_top = 1, size_t pad_bottom = 1, size_t g = 1, bool bias = 0,
                       size_t nt = 1, size_t iter = 10, size_t n = 1);
    ~ConvWinoF63ZCLayer();

    // Grid search over the GEMM tile shapes and the filter-transform strategy;
    // the result stays in the object for Init() (and is appended to the tuning log).
    int Tuning();
    int Init();
    int Forward();

    // Not in the reference: per-output-channel bias (K floats) and ReLU applied
    // inside the output transform.  Call before Init().
    void SetChannelBias(const float *bias_k, bool relu);
    // Not in the reference: fix the tile shape / filter-transform strategy by hand.
    void SetConfig(int gemm_config, int offline_kernel_transform);

    int best_config() const { return gemmConfig_best; }
    int best_offline() const { return scheduling_best % 2; }
    // per-Forward milliseconds of the last Forward(): InputTran, KernelTran, TensorGEMM, OutputTran
    double stage_ms[4] = {0, 0, 0, 0};

    static int DefaultConfig(size_t K, size_t C, size_t H, size_t W, size_t pad, size_t N);

   private:
    fc_conv_shape Shape() const;
    void AllocateFor(int config);
    void RunOnce(bool filter_ready);
    void RunStages(bool filter_ready);

    // blocking of the GEMM stage: the chosen workgroup tile, under the names the
    // reference uses for its cache blocks
    int tileBlock;     // BN: tiles per workgroup
    int ocBlock;       // BM: output channels per workgroup
    int icBlock;       // BK: input channels per LDS stage
    int scheduling;
    int ocRegBlock;    // wavefronts along output channels
    int tileRegBlock;  // wavefronts along tiles
    int enableOffKernel;
    int gemmConfig;

    float *inputBuf;   // V, device
    float *gemmBuf;    // M, device
    float *kernelBuf;  // U, device

    int gemmConfig_best;
    int scheduling_best;

    fc_wino_plan plan;
    LayerDeviceBuffers dev;
    const float *channel_bias;
    bool relu;
};

#endif
