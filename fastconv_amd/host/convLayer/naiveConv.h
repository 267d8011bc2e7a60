// Direct convolution on the host CPU: the checker the driver compares the GPU
// layers with, in the role of the reference's ConvNaiveLayer.  It follows the
// general loop nest (convLayer/naiveConv_wudu.h:48-81: any kernel size, stride
// and padding, per-element bias), of which convLayer/naiveConv.h:24-64 is the
// 3x3 stride-1 case, with the batch as an outer loop and OpenMP over
// (image, output channel).  It is never selected by -a: it only produces
// output_ref.
#pragma once

#include "../conv_layer.h"

class ConvNaiveLayer : public ConvLayer {
   public:
    ConvNaiveLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih, size_t iw,
                   size_t oc, size_t kh = 3, size_t kw = 3, size_t sh = 1, size_t sw = 1, size_t pad_left = 1,
                   size_t pad_right = 1, size_t pad_top = 1, size_t pad_bottom = 1, size_t g = 1, bool bias = 0,
                   size_t nt = 1, size_t iter = 10, size_t n = 1)
        : ConvLayer(input, kernel, biasw, output_ref, ic, ih, iw, oc, kh, kw, sh, sw, pad_left, pad_right, pad_top,
                    pad_bottom, g, bias, nt, iter, n) {}

    int Init() { return -1; }
    int Tuning() { return -1; }

    int Forward() {
        const long output_page = (long)output_height * output_width;
        const long input_page = (long)input_height * input_width;
        const int kernel_page = (int)(kernel_height * kernel_width);
        const long kernel_page_row = (long)input_channels * kernel_page;
        const int OW = (int)output_width, IH = (int)input_height, IW = (int)input_width;
        const int KH = (int)kernel_height, KW = (int)kernel_width;
#pragma omp parallel for collapse(2) schedule(static)
        for (long n = 0; n < (long)batch; n++) {
            for (long oc = 0; oc < (long)output_channels; oc++) {
                const float *xn = input_data + n * (long)input_channels * input_page;
                float *yo = output_data + (n * (long)output_channels + oc) * output_page;
                for (long tile = 0; tile < output_page; tile++) {
                    const int startH = (int)(tile / OW) * (int)stride_height - (int)padding_top;
                    const int startW = (int)(tile % OW) * (int)stride_width - (int)padding_left;
                    float sum = 0;
                    for (long ic = 0; ic < (long)input_channels; ic++) {
                        const float *ip = xn + ic * input_page;
                        const float *kp = kernel_data + oc * kernel_page_row + ic * kernel_page;
                        float total = 0;
                        for (int i = 0; i < KH; i++)
                            for (int j = 0; j < KW; j++) {
                                const int x = startH + i, y = startW + j;
                                if (x < 0 || x >= IH || y < 0 || y >= IW) continue;
                                total += ip[(long)x * IW + y] * kp[i * KW + j];
                            }
                        sum += total;
                    }
                    if (bias_term) sum += bias_data[oc * output_page + tile];
                    yo[tile] = sum;
                }
            }
        }
        return 1;
    }
};
