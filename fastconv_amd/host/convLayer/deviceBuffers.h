// Device-side copies of a layer's input, filter and output, carved from the
// arena; shared by the three GPU layer classes.
#pragma once

#include <stddef.h>

#include "../utility/device.h"

struct LayerDeviceBuffers {
    float *input = NULL, *kernel = NULL, *output = NULL, *bias = NULL;
    size_t mark = 0;
    bool held = false;

    // Remembers the arena offset, then uploads input and filter.
    void Acquire(const float *in, size_t in_elems, const float *k, size_t k_elems, size_t out_elems) {
        fastconv::Device &dev = fastconv::Device::Get();
        mark = dev.Mark();
        held = true;
        input = (float *)dev.Alloc(in_elems * sizeof(float), "input");
        kernel = (float *)dev.Alloc(k_elems * sizeof(float), "kernel");
        output = (float *)dev.Alloc(out_elems * sizeof(float), "output");
        dev.Check(fc_upload(dev.ctx(), input, in, in_elems * sizeof(float)), "upload input");
        dev.Check(fc_upload(dev.ctx(), kernel, k, k_elems * sizeof(float)), "upload kernel");
    }
    void SetBias(const float *bias_host, size_t k) {
        fastconv::Device &dev = fastconv::Device::Get();
        bias = (float *)dev.Alloc(k * sizeof(float), "bias");
        dev.Check(fc_upload(dev.ctx(), bias, bias_host, k * sizeof(float)), "upload bias");
    }
    void Download(float *out_host, size_t out_elems) {
        fastconv::Device &dev = fastconv::Device::Get();
        dev.Check(fc_download(dev.ctx(), out_host, output, out_elems * sizeof(float)), "download output");
    }
    // Gives everything allocated since Acquire() back to the arena.  Layers are
    // released in reverse order of their Init(), as the arena is a stack.
    void Release() {
        if (held) fastconv::Device::Get().Release(mark);
        held = false;
        input = kernel = output = bias = NULL;
    }
};
