// Base class of the convolution layers: same constructor arguments, members and
// Init/Forward/Tuning contract as the reference's ConvLayer (conv_layer.h:24-149),
// plus a trailing batch count `n` (default 1; the reference is batch 1 only).
//
// Ownership is the reference's: the caller keeps the arrays it passes, the layer
// copies input and kernel and frees its copies; output_ref is borrowed.  The
// derived GPU layers upload those copies into the device arena in Init().
#pragma once

#include <assert.h>
#include <omp.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "utility/common.h"
#include "utility/helper.h"

class ConvLayer {
   public:
    ConvLayer(float *input, float *kernel, float *biasw, float *output_ref, size_t ic, size_t ih, size_t iw,
              size_t oc, size_t kh = 3, size_t kw = 3, size_t sh = 1, size_t sw = 1, size_t pad_left = 1,
              size_t pad_right = 1, size_t pad_top = 1, size_t pad_bottom = 1, size_t g = 1, bool bias = 0,
              size_t nt = 1, size_t iter = 10, size_t n = 1) {
        num_threads = nt;
        iterations = iter;
        omp_set_num_threads((int)num_threads);
        batch = n;

        input_channels = ic;
        input_height = ih;
        input_width = iw;
        output_channels = oc;
        kernel_height = kh;
        kernel_width = kw;
        bias_term = bias;
        group = g;
        stride_height = sh;
        stride_width = sw;
        padding_left = pad_left;
        padding_top = pad_top;
        padding_right = pad_right;
        padding_bottom = pad_bottom;
        assert(!(group == 0 || stride_width == 0 || stride_height == 0 || batch == 0));
        if (group != 1) {
            fprintf(stderr, "Error: only group == 1 is supported\n");
            exit(EXIT_FAILURE);
        }
        this->output_ref = output_ref;

        output_width = (input_width + padding_left + padding_right - kernel_width) / stride_width + 1;
        output_height = (input_height + padding_top + padding_bottom - kernel_height) / stride_height + 1;

        const size_t in_elems = batch * input_channels * input_width * input_height;
        const size_t k_elems = input_channels * output_channels * kw * kh;
        const size_t out_elems = batch * output_channels * output_width * output_height;
        input_data = (float *)malloc(in_elems * sizeof(float));
        kernel_data = (float *)malloc((k_elems + 16) * sizeof(float));
        // as in the reference, the bias is one float per output element of one image
        bias_data = (float *)calloc(output_channels * output_width * output_height, sizeof(float));
        output_data = (float *)malloc(out_elems * sizeof(float));
        if (!input_data || !kernel_data || !bias_data || !output_data) {
            fprintf(stderr, "Buffer is NULL.\n");
            exit(EXIT_FAILURE);
        }
        memcpy(input_data, input, in_elems * sizeof(float));
        memcpy(kernel_data, kernel, k_elems * sizeof(float));
        if (biasw) memcpy(bias_data, biasw, output_channels * output_width * output_height * sizeof(float));
    }

    virtual ~ConvLayer() {
        free(input_data);
        free(kernel_data);
        free(bias_data);
        free(output_data);
        input_data = kernel_data = output_data = bias_data = NULL;
    }

    int get_output_height() { return (int)this->output_height; }
    int get_output_width() { return (int)this->output_width; }
    size_t get_batch() { return batch; }
    size_t output_elements() const { return batch * output_channels * output_height * output_width; }
    // direct-convolution FLOP count, the numerator of the effective GFLOP/s
    double flops() const {
        return 2.0 * batch * output_channels * input_channels * output_height * output_width * kernel_height *
               kernel_width;
    }

    virtual int Init() { return -1; }
    virtual int Forward() { return -1; }
    virtual int Tuning() { return -1; }

    // N x K x OH x OW, filled by Forward()
    float *output_data;
    // milliseconds per Forward iteration of the last Forward() call (0 before)
    double last_total_ms = 0.0;

   protected:
    size_t batch;
    size_t input_channels;
    size_t input_width;
    size_t input_height;

    size_t output_channels;
    size_t output_width;
    size_t output_height;

    size_t kernel_width;
    size_t kernel_height;

    size_t stride_width;
    size_t stride_height;

    size_t padding_left;
    size_t padding_right;
    size_t padding_top;
    size_t padding_bottom;

    size_t group;
    bool bias_term;
    size_t num_threads;
    size_t iterations;

    float *input_data;
    float *kernel_data;
    float *bias_data;
    float *output_ref;
};
