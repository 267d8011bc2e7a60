// im2col + GEMM layer, as one implicit-GEMM kernel: the column matrix
// [C*kh*kw] x [N*OH*OW] is never written to memory, each workgroup gathers its
// slice of it into LDS and multiplies on fp32 MFMA.  Interface of the
// reference's ConvIm2colLayer (convLayer/im2colConv.h:9-108): M = output
// channels, N = output pixels, K = C*kh*kw (:23-25); Tuning() -> Init() ->
// Forward().  The CPU blocking arguments of the reference constructor (mc, nc,
// kc, register kernel, prefetch distances) have no meaning on the GPU; the one
// tunable is the workgroup tile shape.
#ifndef IM2COLCONV_H
#define IM2COLCONV_H

#include "../conv_layer.h"
#include "deviceBuffers.h"
#include "fastconv_hip.h"

class ConvIm2colLayer : public ConvLayer {
   public:
    ConvIm2colLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih, size_t iw,
                    size_t oc, size_t kh = 3, size_t kw = 3, size_t sh = 1, size_t sw = 1, size_t pad_left = 1,
                    size_t pad_right = 1, size_t pad_top = 1, size_t pad_bottom = 1, size_t g = 1, bool bias = 0,
                    size_t nt = 1, size_t iter = 10, size_t n = 1, int tile_config = -1);
    ~ConvIm2colLayer();

    int Init();
    int Tuning();
    int Forward();

    void SetChannelBias(const float *bias_k, bool relu);
    int best_config() const { return config_best; }
    double gemm_ms = 0.0;   // per-Forward milliseconds of the implicit-GEMM kernel in the last Forward()

   protected:
    int M;
    long N;
    int K;
    int config;
    int config_best;

    fc_conv_shape Shape() const;
    void AllocateFor(int cfg);
    void RunOnce();

    float *packed_kernel;   // Wp[Kred_pad][K_pad], device
    int32_t *gather_table;  // device
    float *workspace;       // device, partial sums when the plan splits the reduction
    fc_igemm_plan plan;
    LayerDeviceBuffers dev;
    const float *channel_bias;
    bool relu;
};

#endif
