// Host-side helpers of the layer classes: wall-clock Timer, the legacy diff()
// self-check and the option enums of the ConvTest driver.  Same names and
// meaning as the reference's utility/helper.h:66-126 so that driver and layer
// code read the same; nothing here touches the GPU.
#pragma once

#include <stddef.h>
#include <stdio.h>
#include <time.h>

#define LOGI(...) fprintf(stdout, __VA_ARGS__)
#define LOGD(...) fprintf(stdout, __VA_ARGS__)
#define LOGE(...) fprintf(stderr, __VA_ARGS__)

// Mean absolute difference over the elements that differ by more than 1e-5
// (1e-4 for the 2-D form); prints "The difference is ..." and returns it
// (utility/helper.cpp:74-109).
float diff(float *arr1, float *arr2, int len);
float diff(float *arr1, float *arr2, int M, int N);

// max_i |y_i - ref_i| / max_i |ref_i|: the scale-normalised error the
// tolerance gates are stated in (im2col 1e-5, Winograd 1e-3).
double max_rel_err(const float *y, const float *ref, size_t len);

class Timer {
   public:
    Timer() : accumulate(0) {}
    virtual ~Timer() {}
    void startBench();
    void accumBench();
    void printBench(const char *comments, int fold);
    void endBench(const char *comments);
    void endBench(const char *comments, double fold);
    double endBench(double fold);
    double accumulated() const { return accumulate; }

   private:
    timespec start, stop;
    double accumulate;
};

struct nnp_size {
    size_t width;
    size_t height;
};

struct nnp_padding {
    size_t top;
    size_t right;
    size_t bottom;
    size_t left;
};

enum nnp_convolution_algorithm {
    nnp_convolution_algorithm_auto = 0,
    nnp_convolution_algorithm_direct = 1,    // 1x1 stride 1: the implicit-GEMM kernel without window arithmetic
    nnp_convolution_algorithm_im2col = 2,    // implicit GEMM (no column matrix in memory)
    nnp_convolution_algorithm_winograd = 3   // F(6x6, 3x3), 3x3 stride 1 only
};

enum nnp_convolution_transform_strategy {
    nnp_convolution_transform_strategy_online = 0,    // filter transform inside every Forward
    nnp_convolution_transform_strategy_offline = 1,   // filter transform once in Init
};

enum nnp_convolution_tuning_strategy {
    nnp_convolution_tuning_strategy_no_tuning = 0,
    nnp_convolution_tuning_strategy_grid_search = 1,
};
