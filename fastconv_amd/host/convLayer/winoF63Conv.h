// Winograd F(6x6,3x3) layer, blocked pipeline: the GEMM result of one block of
// (32 output channels x 32 tiles x 64 frequencies) is consumed by the output
// transform straight out of registers and LDS -- there is no whole-layer M
// buffer -- and the batch may be cut into blocks of `tileBlock` tiles (whole
// images) so that only one block of V exists at a time.  The filter transform runs
// in every Forward() pass (online, the default) or once in Init() (offline:
// SetConfig(..., 1), or chosen by Tuning()).  Interface of the reference's ConvWinoF63Layer
// (convLayer/winoF63Conv.h:4-209), whose scratch is likewise sized for one
// (ocBlock x tileBlock) block and whose GEMM output goes to the output
// transform through a small buffer (winoF63/winoF63.cpp:1574-1737).
#ifndef WINOF63CONV_H_
#define WINOF63CONV_H_

#include "../conv_layer.h"
#include "../utility/helper.h"
#include "deviceBuffers.h"
#include "fastconv_hip.h"

class ConvWinoF63Layer : public ConvLayer {
   public:
    ConvWinoF63Layer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih, size_t iw,
                     size_t oc, size_t kh = 3, size_t kw = 3, size_t sh = 1, size_t sw = 1, size_t pad_left = 1,
                     size_t pad_right = 1, size_t pad_top = 1, size_t pad_bottom = 1, size_t g = 1, bool bias = 0,
                     size_t nt = 1, size_t iter = 10, size_t n = 1);
    ~ConvWinoF63Layer();

    int Tuning();
    int Init();
    int Forward();

    void SetChannelBias(const float *bias_k, bool relu);
    // Not in the reference: fix tile shape and images per block by hand (0 images per block: the
    // single-kernel engine over the whole batch).
    void SetConfig(int gemm_config, int images_per_block);
    void SetOfflineKernelTransform(bool offline) { enableOffKernel_best = offline ? 1 : 0; }
    int best_config() const { return gemmConfig_best; }
    int best_offline() const { return enableOffKernel_best; }
    int best_images_per_block() const { return imgBlock_best; }
    double stage_ms[4] = {0, 0, 0, 0};

    // Images per block whose V and M scratch is about `budget_bytes`.
    static int DefaultImagesPerBlock(size_t K, size_t C, size_t tiles_per_image, size_t N, size_t budget_bytes);

   private:
    fc_conv_shape Shape(int n) const;
    void AllocateFor(int config, int images_per_block);
    void RunOnce(bool split_stages = false);

    int tileBlock;   // tiles per block = images per block x tiles per image
    int ocBlock;     // BM of the GEMM tile
    int icBlock;     // BK of the GEMM tile
    int ocRegBlock;
    int tileRegBlock;
    int enableOffKernel;
    int imgBlock;

    float *inputBuf;    // V of one block, device
    float *gemmBuf;     // unused: the products never leave the compute unit
    float *kernelBuf;   // U of the whole layer, device

    int gemmConfig_best;
    int imgBlock_best;
    int enableOffKernel_best;

    fc_wino_plan plan, tailPlan;   // full blocks / the last partial block
    bool hasTail;
    bool onePass;      // images per block 0: input transform, products and output transform in one kernel
    LayerDeviceBuffers dev;
    const float *channel_bias;
    bool relu;
};

#endif
