// Runs a VGG-16 style convolution trunk (13 x [3x3 conv + bias + ReLU], 2x2 max pooling
// between the blocks) back to back on the device through the layer graph of layer.h, and
// checks the result against the same chain on the host (ConvNaiveLayer + ReLU + pooling).
//   net_test [-n batch] [-is size] [-w width_divisor] [-i iterations] [--no-check] [--graph]
// --graph records the trunk once and replays the recording (one launch call per forward pass).
// -w 4 divides every channel count by 4 (a small trunk whose host check takes seconds).
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <vector>

#include "convLayer/naiveConv.h"
#include "layer.h"
#include "utility/device.h"
#include "utility/helper.h"
#include "utility/rng.h"

int main(int argc, char **argv) {
    size_t batch = 1, size = 32, divisor = 4, iterations = 5;
    bool check = true, graph = false;
    for (int i = 1; i < argc; i++) {
        if (!strcmp(argv[i], "-n") && i + 1 < argc) batch = strtoul(argv[++i], NULL, 10);
        else if (!strcmp(argv[i], "-is") && i + 1 < argc) size = strtoul(argv[++i], NULL, 10);
        else if (!strcmp(argv[i], "-w") && i + 1 < argc) divisor = strtoul(argv[++i], NULL, 10);
        else if (!strcmp(argv[i], "-i") && i + 1 < argc) iterations = strtoul(argv[++i], NULL, 10);
        else if (!strcmp(argv[i], "--no-check")) check = false;
        else if (!strcmp(argv[i], "--graph")) graph = true;
        else { fprintf(stderr, "Error: unknown argument '%s'\n", argv[i]); return 1; }
    }
    if (batch == 0 || size < 32 || size % 32 || divisor == 0 || 64 % divisor) {
        fprintf(stderr, "Error: need batch > 0, an input size that is a multiple of 32, a divisor of 64\n");
        return 1;
    }
    const int cfg[] = {64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512};
    const int ncfg = sizeof cfg / sizeof cfg[0];

    // weights and input
    std::vector<std::vector<float> > weights, biases;
    size_t c = 3;
    double flops = 0;
    size_t h = size;
    for (int i = 0; i < ncfg; i++) {
        if (cfg[i] < 0) { h /= 2; continue; }
        const size_t k = cfg[i] / divisor;
        std::vector<float> w(k * c * 9), b(k);
        fastconv::FillNormal(100 + i, (float)sqrt(2.0 / (9.0 * c)), w.data(), w.size());
        fastconv::FillUniform(200 + i, -0.1f, 0.1f, b.data(), b.size());
        weights.push_back(w);
        biases.push_back(b);
        flops += 2.0 * batch * k * c * h * h * 9;
        c = k;
    }
    std::vector<float> input(batch * 3 * size * size);
    fastconv::FillUniform(1, -1.f, 1.f, input.data(), input.size());

    // device graph
    size_t arena = (size_t)256 << 20;
    arena += batch * size * size * (64 / divisor) * 4 * 40;            // activations
    arena += batch * ((size + 5) / 6) * ((size + 5) / 6) * 256 * 2 * (128 / divisor + 32) + ((size_t)1 << 28);
    fastconv::Device::Configure(arena + ((size_t)64 << 20));
    feather::Net net(arena);
    net.SetInput(batch, 3, size, size);
    int li = 0;
    for (int i = 0; i < ncfg; i++) {
        char name[32];
        if (cfg[i] < 0) {
            snprintf(name, sizeof name, "pool%d", i);
            net.Add(new feather::MaxPool2x2Layer(name));
        } else {
            snprintf(name, sizeof name, "conv%d", li);
            net.Add(new feather::ConvolutionLayer(name, cfg[i] / divisor, 3, 1, 1, weights[li].data(), biases[li].data(), true));
            li++;
        }
    }
    if (net.Init() != 0) return 1;
    printf("Layer graph: %zu layers, shared scratch %zu KB, direct-convolution FLOP count %.3f GFLOP\n", net.num_layers(),
           net.common_bytes() / 1024, flops / 1e9);
    fastconv::Device &d = fastconv::Device::Get();
    net.Forward(input.data());
    d.Check(fc_sync(d.ctx()), "fc_sync");
    if (graph) {
        if (net.RecordGraph() != 0) return 1;
        printf("Forward passes replay a recorded graph\n");
        // the checked result below comes from a replay on fresh input, not from the eager pass
        std::vector<float> other(input.size());
        fastconv::FillUniform(2, -1.f, 1.f, other.data(), other.size());
        net.Forward(other.data());
        net.Forward(input.data());
        d.Check(fc_sync(d.ctx()), "fc_sync");
    }
    Timer t;
    t.startBench();
    for (size_t i = 0; i < iterations; i++) net.Forward(NULL);
    d.Check(fc_sync(d.ctx()), "fc_sync");
    const double ms = t.endBench((double)iterations);
    printf("Total time: %lfms\n", ms);
    printf("Effective GFLOP/s: %.1f\n", flops / (ms * 1e-3) / 1e9);
    const feather::Blob<float> *out = net.output();
    std::vector<float> y(out->data_size());
    out->CopyToHost(y.data());

    int status = 0;
    if (check) {
        // the same chain on the host: naive conv + bias + ReLU, 2x2 max pooling
        std::vector<float> cur = input;
        size_t ch = 3, hh = size;
        li = 0;
        for (int i = 0; i < ncfg; i++) {
            if (cfg[i] < 0) {
                std::vector<float> nxt(batch * ch * (hh / 2) * (hh / 2));
                for (size_t pl = 0; pl < batch * ch; pl++)
                    for (size_t a = 0; a < hh / 2; a++)
                        for (size_t b = 0; b < hh / 2; b++) {
                            const float *s = &cur[(pl * hh + 2 * a) * hh + 2 * b];
                            nxt[(pl * (hh / 2) + a) * (hh / 2) + b] = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[hh], s[hh + 1]));
                        }
                cur.swap(nxt);
                hh /= 2;
                continue;
            }
            const size_t k = cfg[i] / divisor;
            ConvNaiveLayer ref(cur.data(), weights[li].data(), NULL, NULL, ch, hh, hh, k, 3, 3, 1, 1, 1, 1, 1, 1, 1, false, 16,
                               1, batch);
            ref.Forward();
            std::vector<float> nxt(batch * k * hh * hh);
            for (size_t n = 0; n < batch; n++)
                for (size_t kk = 0; kk < k; kk++)
                    for (size_t px = 0; px < hh * hh; px++) {
                        const size_t idx = (n * k + kk) * hh * hh + px;
                        nxt[idx] = fmaxf(ref.output_data[idx] + biases[li][kk], 0.f);
                    }
            cur.swap(nxt);
            ch = k;
            li++;
        }
        const double err = max_rel_err(y.data(), cur.data(), y.size());
        const bool ok = err <= 1e-3 && y.size() == cur.size();
        printf("Max relative error vs host chain: %.3e (tolerance 1e-03) %s\n", err, ok ? "PASS" : "FAIL");
        if (!ok) status = 2;
    }
    return status;
}
