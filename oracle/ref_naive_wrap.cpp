/*
 * C entry points around the reference's own naive convolution layers, compiled
 * from the reference headers where they lie (see oracle/Makefile, target
 * `ref`).  TEST INFRASTRUCTURE ONLY.  No reference source is copied here: the
 * two headers are included by path, each inside its own namespace because both
 * name their class ConvNaiveLayer.
 *
 *   ref_naive_3x3s1   convLayer/naiveConv.h:24-64   (3x3, stride 1, any pad)
 *   ref_naive_general convLayer/naiveConv_wudu.h:48-81 (any kernel/stride/pad,
 *                     adds a per-element bias tensor of K*OH*OW floats)
 *
 * The reference has no batch dimension; callers loop over images.
 */
#include "conv_layer.h"

namespace ref_fixed3x3 {
#include "convLayer/naiveConv.h"
}
namespace ref_general {
#include "convLayer/naiveConv_wudu.h"
}

#include <cstring>
#include <vector>

extern "C" {

int ref_naive_3x3s1(const float *x, const float *w, float *y, int C, int H, int W, int K,
                    int pad_l, int pad_r, int pad_t, int pad_b) {
    ref_fixed3x3::ConvNaiveLayer layer(const_cast<float *>(x), const_cast<float *>(w), NULL, NULL,
                                       C, H, W, K, 3, 3, 1, 1, pad_l, pad_r, pad_t, pad_b);
    const int rc = layer.Forward();
    const size_t n = (size_t)K * layer.get_output_height() * layer.get_output_width();
    std::memcpy(y, layer.output_data, n * sizeof(float));
    return rc;
}

/* bias_elems: K*OH*OW floats added per output element, or NULL for zero. */
int ref_naive_general(const float *x, const float *w, const float *bias_elems, float *y,
                      int C, int H, int W, int K, int kh, int kw, int sh, int sw,
                      int pad_l, int pad_r, int pad_t, int pad_b) {
    const int OW = (W + pad_l + pad_r - kw) / sw + 1;
    const int OH = (H + pad_t + pad_b - kh) / sh + 1;
    const size_t n = (size_t)K * OH * OW;
    /* The base constructor always allocates the bias tensor and fills it only
     * when one is passed; hand it zeros so the sum is defined. */
    std::vector<float> zeros;
    const float *b = bias_elems;
    if (!b) { zeros.assign(n, 0.f); b = zeros.data(); }
    ref_general::ConvNaiveLayer layer(const_cast<float *>(x), const_cast<float *>(w),
                                      const_cast<float *>(b), NULL, C, H, W, K, kh, kw, sh, sw,
                                      pad_l, pad_r, pad_t, pad_b, 1, true);
    const int rc = layer.Forward();
    std::memcpy(y, layer.output_data, n * sizeof(float));
    return rc;
}

}  /* extern "C" */
