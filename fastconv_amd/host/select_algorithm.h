// Algorithm choice for `-a auto`.  The reference picks by kernel size and
// stride alone (ConvTest.cpp:318-331: 1x1 stride 1 -> direct, 3x3 stride 1 ->
// winograd, otherwise im2col).  The same skeleton is kept, with the 3x3
// stride-1 case refined by what was measured on MI355X: the staged Winograd
// pipeline moves 64 planes of V and M per layer, which only pays when there is
// enough arithmetic per plane element.
#pragma once

#include <algorithm>

#include "utility/helper.h"

inline enum nnp_convolution_algorithm select_algorithm(struct nnp_size kernel_size, struct nnp_size output_subsampling,
                                                       struct nnp_size output_size, size_t input_channels,
                                                       size_t output_channels, size_t batch) {
    if (std::max(output_subsampling.height, output_subsampling.width) == 1) {
        if (std::max(kernel_size.height, kernel_size.width) == 1) {
            return nnp_convolution_algorithm_direct;
        } else if (kernel_size.height == 3 && kernel_size.width == 3) {
            const size_t tiles = batch * ((output_size.height + 5) / 6) * ((output_size.width + 5) / 6);
            // few input channels: the M planes (64 floats per 36 outputs) dominate and carry no reuse
            if (input_channels < 16) return nnp_convolution_algorithm_im2col;
            // few tiles: the 64x larger transformed filter dominates
            if (tiles < 64 && input_channels * output_channels >= 128 * 128) return nnp_convolution_algorithm_im2col;
            return nnp_convolution_algorithm_winograd;
        }
    }
    return nnp_convolution_algorithm_im2col;
}
