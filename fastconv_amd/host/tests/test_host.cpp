// Unit tests of the host-side logic that needs no GPU: the range allocator under
// the memory pools, the pools themselves (over a made-up base address: nothing is
// dereferenced), the tuning log, the algorithm choice and the output-size
// arithmetic of ConvLayer.  Exit status 0 = all passed.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <unistd.h>

#include "conv_layer.h"
#include "convLayer/naiveConv.h"
#include "select_algorithm.h"
#include "utility/mempool.h"
#include "utility/range_allocator.h"
#include "utility/rng.h"
#include "utility/tuning_log.h"

static int failures = 0;
#define CHECK(cond)                                                      \
    do {                                                                 \
        if (!(cond)) {                                                   \
            fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            failures++;                                                  \
        }                                                                \
    } while (0)

static void test_range_allocator() {
    char *base = (char *)0x7f0000000000ULL;          // never dereferenced
    fastconv::RangeAllocator a(base, 4096, 256);
    void *p1 = a.Allocate(100), *p2 = a.Allocate(300), *p3 = a.Allocate(256);
    CHECK(p1 == base && p2 == base + 256 && p3 == base + 768);
    CHECK(a.used() == 256 + 512 + 256 && a.live_blocks() == 3);
    CHECK(a.Allocate(4096) == NULL);                 // does not fit
    CHECK(a.Allocate(0) == NULL);
    CHECK(a.Free(p2));
    CHECK(!a.Free(p2));                              // double free is reported
    CHECK(!a.Free(base + 8));                        // foreign pointer is reported
    void *p4 = a.Allocate(512);                      // first fit reuses the hole
    CHECK(p4 == p2);
    CHECK(a.Free(p1) && a.Free(p4) && a.Free(p3));
    CHECK(a.used() == 0 && a.free_blocks() == 1 && a.largest_free() == 4096);   // fully coalesced
    CHECK(a.peak() == 1024);
    void *all = a.Allocate(4096);
    CHECK(all == base && a.Allocate(1) == NULL);
}

static void test_pools() {
    char *base = (char *)0x7e0000000000ULL;
    fastconv::RangeAllocator a(base, 1 << 20, 256);
    CommonMemPool<float> common(&a);
    float *ptr = NULL;
    CHECK(!common.GetPtr(&ptr));                     // nothing allocated yet
    CHECK(common.Request(1000) && common.Request(5000) && common.Request(200));
    CHECK(common.common_bytes() == 5000);            // the largest request wins
    CHECK(common.Request(300, 7) && common.Request(100, 7) && common.Request(64, 9));
    CHECK(common.Alloc());
    CHECK(!common.Alloc());                          // already allocated
    CHECK(common.GetPtr(&ptr) && ptr != NULL);
    float *p7 = NULL, *p9 = NULL, *pbad = NULL;
    CHECK(common.GetPtr(&p7, 7) && common.GetPtr(&p9, 9) && p7 != p9 && p7 != ptr);
    CHECK(!common.GetPtr(&pbad, 8));
    CHECK(a.SizeOf(p7) == 512 && a.SizeOf(ptr) == 5120);
    CHECK(common.Free(7) && !common.Free(7));
    CHECK(common.Alloc(9000));                       // grows the default pool
    CHECK(common.GetPtr(&ptr) && a.SizeOf(ptr) == 9216);
    CHECK(common.FreeAll() && a.used() == 0);

    PrivateMemPool<float> priv(&a);
    float *q1 = NULL, *q2 = NULL;
    size_t sz = 0;
    CHECK(priv.Alloc(&q1, 1024) && priv.Alloc(&q2, 4096) && q1 != q2);
    CHECK(priv.GetSize(q2, &sz) && sz == 4096);
    float *stray = (float *)(base + 12345);
    CHECK(!priv.GetSize(stray, &sz) && !priv.Free(&stray));
    CHECK(priv.Free(&q1) && q1 == NULL && priv.count() == 1);
    float *big = NULL;
    CHECK(!priv.Alloc(&big, (size_t)2 << 20) && big == NULL);   // exhaustion: false, not a crash
    CHECK(priv.FreeAll() && a.used() == 0);
}

static void test_tuning_log() {
    char path[] = "/tmp/fastconv_tlog_XXXXXX";
    int fd = mkstemp(path);
    CHECK(fd >= 0);
    close(fd);
    setenv("FASTCONV_TUNING_LOG", path, 1);
    TuningKey k1 = {"winograd_zc", 32, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1};
    TuningKey k2 = {"im2col", 1, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1};
    TuningEntry e;
    CHECK(!tuning_log_lookup(k1, &e));
    TuningEntry a = {5, 1, 0.4321}, b = {0, 0, 0.3999}, c = {3, 0, 0.05};
    CHECK(tuning_log_append(k1, a) && tuning_log_append(k2, c) && tuning_log_append(k1, b));
    CHECK(tuning_log_lookup(k1, &e) && e.config == 0 && e.option == 0 && fabs(e.ms - 0.3999) < 1e-9);  // last wins
    CHECK(tuning_log_lookup(k2, &e) && e.config == 3);
    TuningKey k3 = k1;
    k3.n = 3;                                        // "3,..." must not match the "32,..." line
    CHECK(!tuning_log_lookup(k3, &e));
    unlink(path);
    unsetenv("FASTCONV_TUNING_LOG");
}

static void test_select_algorithm() {
    nnp_size k3 = {3, 3}, k1 = {1, 1}, k7 = {7, 7}, s1 = {1, 1}, s2 = {2, 2};
    nnp_size o56 = {56, 56}, o224 = {224, 224};
    // the reference's skeleton (ConvTest.cpp:318-331)
    CHECK(select_algorithm(k1, s1, o56, 64, 256, 1) == nnp_convolution_algorithm_direct);
    CHECK(select_algorithm(k3, s2, o56, 256, 256, 32) == nnp_convolution_algorithm_im2col);
    CHECK(select_algorithm(k1, s2, o56, 256, 512, 1) == nnp_convolution_algorithm_im2col);
    CHECK(select_algorithm(k7, s2, o224, 3, 64, 1) == nnp_convolution_algorithm_im2col);
    // 3x3 stride 1: the rule must pick the measured winner on every VGG-16 / ResNet-50 layer at batch 1, 4
    // and 32 and on the ResNet-50 layers at batch 8 and 16, where the two algorithms cross (whole-layer
    // milliseconds on MI355X, Winograd and implicit GEMM at their best tile shape);
    // layers where the two are within 15 % of each other may go either way (boxes of the pool differ by up to that
    // much on layers bound by their stores, such as the 3-channel first layer)
    static const struct { int c, k, h, n; double wino_ms, im2col_ms; } measured[] = {
        {3, 64, 224, 1, 0.0203, 0.0117}, {64, 64, 224, 1, 0.0367, 0.0486}, {64, 128, 112, 1, 0.0301, 0.0302},
        {128, 128, 112, 1, 0.0330, 0.0491}, {128, 256, 56, 1, 0.0304, 0.0284}, {256, 256, 56, 1, 0.0341, 0.0469},
        {256, 512, 28, 1, 0.0268, 0.0277}, {512, 512, 28, 1, 0.0341, 0.0463}, {512, 512, 14, 1, 0.0302, 0.0190},
        {64, 64, 56, 1, 0.0198, 0.0107}, {128, 128, 28, 1, 0.0193, 0.0105}, {256, 256, 14, 1, 0.0214, 0.0107},
        {512, 512, 7, 1, 0.0307, 0.0141}, {3, 64, 224, 4, 0.0332, 0.0217}, {64, 64, 224, 4, 0.0922, 0.1397},
        {64, 128, 112, 4, 0.0465, 0.0802}, {128, 128, 112, 4, 0.0628, 0.1381}, {128, 256, 56, 4, 0.0418, 0.0798},
        {256, 256, 56, 4, 0.0587, 0.1428}, {256, 512, 28, 4, 0.0447, 0.0809}, {512, 512, 28, 4, 0.0683, 0.1505},
        {512, 512, 14, 4, 0.0474, 0.0468}, {64, 64, 56, 4, 0.0256, 0.0194}, {128, 128, 28, 4, 0.0253, 0.0185},
        {256, 256, 14, 4, 0.0290, 0.0192}, {512, 512, 7, 4, 0.0313, 0.0190}, {64, 64, 56, 8, 0.0322, 0.0309},
        {128, 128, 28, 8, 0.0306, 0.0284}, {256, 256, 14, 8, 0.0372, 0.0274}, {512, 512, 7, 8, 0.0361, 0.0296},
        {64, 64, 56, 16, 0.0368, 0.0474}, {128, 128, 28, 16, 0.0360, 0.0478}, {256, 256, 14, 16, 0.0415, 0.0464},
        {512, 512, 7, 16, 0.0519, 0.0467}, {3, 64, 224, 32, 0.1206, 0.1312}, {64, 64, 224, 32, 0.4979, 1.0260},
        {64, 128, 112, 32, 0.2675, 0.4769}, {128, 128, 112, 32, 0.4275, 0.9476}, {128, 256, 56, 32, 0.1979, 0.4817},
        {256, 256, 56, 32, 0.3231, 0.9416}, {256, 512, 28, 32, 0.1670, 0.4903}, {512, 512, 28, 32, 0.2932, 0.9387},
        {512, 512, 14, 32, 0.1314, 0.2724}, {64, 64, 56, 32, 0.0538, 0.0797}, {128, 128, 28, 32, 0.0459, 0.0781},
        {256, 256, 14, 32, 0.0533, 0.0798}, {512, 512, 7, 32, 0.0741, 0.0835}};
    for (size_t i = 0; i < sizeof measured / sizeof measured[0]; i++) {
        const nnp_size o = {(size_t)measured[i].h, (size_t)measured[i].h};
        const bool wino = select_algorithm(k3, s1, o, measured[i].c, measured[i].k, measured[i].n) == nnp_convolution_algorithm_winograd;
        const double ratio = measured[i].wino_ms / measured[i].im2col_ms;
        if (ratio < 1.0 / 1.15) CHECK(wino);
        if (ratio > 1.15) CHECK(!wino);
    }
    // wider than the Winograd input transform admits: implicit GEMM
    nnp_size wide = {1021, 9};      // {width, height}
    CHECK(select_algorithm(k3, s1, wide, 64, 64, 8) == nnp_convolution_algorithm_im2col);
}

static void test_conv_layer_geometry_and_naive() {
    // 8 channels of ones, 9x9, 3x3 kernel of ones, stride 2, pad 1: corner 32, centre 72
    const int C = 8, H = 9, K = 2;
    float *x = (float *)malloc(sizeof(float) * 2 * C * H * H), *w = (float *)malloc(sizeof(float) * K * C * 9);
    for (int i = 0; i < 2 * C * H * H; i++) x[i] = 1.f;
    for (int i = 0; i < K * C * 9; i++) w[i] = 1.f;
    ConvNaiveLayer layer(x, w, NULL, NULL, C, H, H, K, 3, 3, 2, 2, 1, 1, 1, 1, 1, false, 2, 1, 2);
    CHECK(layer.get_output_height() == 5 && layer.get_output_width() == 5 && layer.get_batch() == 2);
    CHECK(layer.output_elements() == 2u * K * 25);
    CHECK(layer.flops() == 2.0 * 2 * K * C * 25 * 9);
    CHECK(layer.Forward() == 1);
    CHECK(layer.output_data[0] == 32.f && layer.output_data[2 * 5 + 2] == 72.f);
    CHECK(layer.output_data[(1 * K + 1) * 25 + 12] == 72.f);      // second image, second channel, centre
    CHECK(layer.Init() == -1 && layer.Tuning() == -1);            // the reference's return codes
    // legacy diff(): mean of the differences above 1e-5
    float a[4] = {1, 2, 3, 4}, b[4] = {1, 2.5f, 3, 3};
    CHECK(fabsf(diff(a, b, 4) - 0.75f) < 1e-6f && diff(a, a, 4) == 0.f);
    CHECK(fabs(max_rel_err(b, a, 4) - 0.25) < 1e-12);
    free(x);
    free(w);
}

static void test_rng() {
    float u[1000], g[1001];
    fastconv::FillUniform(7, -1.f, 1.f, u, 1000);
    double s = 0;
    for (int i = 0; i < 1000; i++) {
        CHECK(u[i] >= -1.f && u[i] < 1.f);
        s += u[i];
    }
    CHECK(fabs(s / 1000) < 0.1);
    fastconv::FillNormal(7, 0.5f, g, 1001);
    double m = 0, v = 0;
    for (int i = 0; i < 1001; i++) m += g[i];
    m /= 1001;
    for (int i = 0; i < 1001; i++) v += (g[i] - m) * (g[i] - m);
    CHECK(fabs(m) < 0.1 && fabs(sqrt(v / 1001) - 0.5) < 0.05);
    if (getenv("FASTCONV_DUMP_RNG")) {               // lets the Python test compare bit patterns with the oracle
        for (int i = 0; i < 8; i++) printf("U %a\n", u[i]);
        for (int i = 0; i < 8; i++) printf("G %a\n", g[i]);
    }
}

// `test_host --naive in.bin out.bin`: runs the host ConvNaiveLayer on a case read from in.bin
// (13 int32 of geometry N,C,H,W,K,kh,kw,sh,sw,pt,pb,pl,pr, one int32 "has per-element bias",
// then x, w and the optional bias as float32) and writes the output as float32, so that a
// test can compare its bits with stored results of the reference's own naive layers.
static int run_naive_case(const char *in_path, const char *out_path) {
    FILE *f = fopen(in_path, "rb");
    if (!f) return 2;
    int g[14];
    if (fread(g, sizeof(int), 14, f) != 14) return 2;
    const size_t N = g[0], C = g[1], H = g[2], W = g[3], K = g[4], kh = g[5], kw = g[6];
    const size_t nx = N * C * H * W, nw = K * C * kh * kw;
    const size_t OH = (H + g[9] + g[10] - kh) / g[7] + 1, OW = (W + g[11] + g[12] - kw) / g[8] + 1;
    float *x = (float *)malloc(sizeof(float) * nx), *w = (float *)malloc(sizeof(float) * nw), *b = NULL;
    if (fread(x, sizeof(float), nx, f) != nx || fread(w, sizeof(float), nw, f) != nw) return 2;
    if (g[13]) {
        b = (float *)malloc(sizeof(float) * K * OH * OW);
        if (fread(b, sizeof(float), K * OH * OW, f) != K * OH * OW) return 2;
    }
    fclose(f);
    ConvNaiveLayer layer(x, w, b, NULL, C, H, W, K, kh, kw, g[7], g[8], g[11], g[12], g[9], g[10], 1, b != NULL, 2, 1, N);
    layer.Forward();
    FILE *o = fopen(out_path, "wb");
    if (!o) return 2;
    fwrite(layer.output_data, sizeof(float), layer.output_elements(), o);
    fclose(o);
    free(x);
    free(w);
    free(b);
    return 0;
}

int main(int argc, char **argv) {
    if (argc == 4 && strcmp(argv[1], "--naive") == 0) return run_naive_case(argv[2], argv[3]);
    test_range_allocator();
    test_pools();
    test_tuning_log();
    test_select_algorithm();
    test_conv_layer_geometry_and_naive();
    test_rng();
    if (failures) {
        fprintf(stderr, "%d check(s) failed\n", failures);
        return 1;
    }
    printf("all host tests passed\n");
    return 0;
}
