// Winograd F(6x6,3x3) layer, blocked pipeline: the batch is cut into blocks of
// `tileBlock` tiles (whole images) and the input transform, GEMM and output
// transform run block after block over block-local V and M scratch, so the
// 64-plane intermediates of one block stay in the 256 MB memory-side cache
// instead of making a round trip through HBM.  The filter transform is always
// done once in Init().  Interface of the reference's ConvWinoF63Layer
// (convLayer/winoF63Conv.h:4-209), whose scratch is likewise sized for one
// (ocBlock x tileBlock) block (:161-166).
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
    // Not in the reference: fix tile shape and images per block by hand.
    void SetConfig(int gemm_config, int images_per_block);
    int best_config() const { return gemmConfig_best; }
    int best_images_per_block() const { return imgBlock_best; }
    double stage_ms[4] = {0, 0, 0, 0};

    // Images per block whose V and M scratch is about `budget_bytes`.
    static int DefaultImagesPerBlock(size_t K, size_t C, size_t tiles_per_image, size_t N, size_t budget_bytes);

   private:
    fc_conv_shape Shape(int n) const;
    void AllocateFor(int config, int images_per_block);
    void RunOnce();

    int tileBlock;   // tiles per block = images per block x tiles per image
    int ocBlock;     // BM of the GEMM tile
    int icBlock;     // BK of the GEMM tile
    int ocRegBlock;
    int tileRegBlock;
    int enableOffKernel;
    int imgBlock;

    float *inputBuf;    // V of one block, device
    float *gemmBuf;     // M of one block, device
    float *kernelBuf;   // U of the whole layer, device

    int gemmConfig_best;
    int imgBlock_best;

    fc_wino_plan plan, tailPlan;   // full blocks / the last partial block
    bool hasTail;
    LayerDeviceBuffers dev;
    const float *channel_bias;
    bool relu;
};

#endif
