// Algorithm choice for `-a auto`.  The reference picks by kernel size and
// stride alone (ConvTest.cpp:318-331: 1x1 stride 1 -> direct, 3x3 stride 1 ->
// winograd, otherwise im2col).  The same skeleton is kept; the 3x3 stride-1 case
// asks the kernel library, whose rule (fc_prefer_winograd) is derived from
// measured per-layer times of both paths on MI355X.
#pragma once

#include <algorithm>

#include "fastconv_hip.h"
#include "utility/helper.h"

inline enum nnp_convolution_algorithm select_algorithm(struct nnp_size kernel_size, struct nnp_size output_subsampling,
                                                       struct nnp_size output_size, size_t input_channels,
                                                       size_t output_channels, size_t batch) {
    if (std::max(output_subsampling.height, output_subsampling.width) == 1) {
        if (std::max(kernel_size.height, kernel_size.width) == 1) {
            return nnp_convolution_algorithm_direct;
        } else if (kernel_size.height == 3 && kernel_size.width == 3) {
            // the rule sees the layer through its output size: an input of the same size with padding 1
            fc_conv_shape s = {(int)batch, (int)input_channels, (int)output_size.height, (int)output_size.width,
                               (int)output_channels, 3, 3, 1, 1, 1, 1, 1, 1};
            return fc_prefer_winograd(&s) ? nnp_convolution_algorithm_winograd : nnp_convolution_algorithm_im2col;
        }
    }
    return nnp_convolution_algorithm_im2col;
}
