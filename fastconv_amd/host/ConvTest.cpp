// Single-layer convolution driver: builds one random conv layer from the command
// line, computes the naive reference on the host, then runs the chosen GPU
// algorithm and prints per-stage milliseconds, effective GFLOP/s and the error
// against the naive result.  Flags of the reference driver (ConvTest.cpp:92-316)
// keep their names and meaning; --batch, --seed, --variant, --no-check, --strict
// and --json are additions.
#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include <algorithm>

#include "conv_layer.h"
#include "convLayer/im2colConv.h"
#include "convLayer/naiveConv.h"
#include "convLayer/winoF63Conv.h"
#include "convLayer/winoF63ConvZC.h"
#include "select_algorithm.h"
#include "utility/device.h"
#include "utility/helper.h"
#include "utility/rng.h"

// Input uniform in [-1, 1) (the reference draws 256*rand()/RAND_MAX, ConvTest.cpp:18-30).
void fillTestInput(float *target, size_t batch, int inChannels, nnp_size inputDim, uint64_t seed) {
    fastconv::FillUniform(seed * 2 + 1, -1.f, 1.f, target, batch * inChannels * inputDim.height * inputDim.width);
}

// He-normal weights, sigma = sqrt(2 / (kh*kw*C)) (the reference draws rand()/RAND_MAX, ConvTest.cpp:32-46).
void fillTestKernel(float *target, int inChannels, int outChannels, nnp_size kernelDim, uint64_t seed) {
    const float sigma = (float)sqrt(2.0 / ((double)kernelDim.height * kernelDim.width * inChannels));
    fastconv::FillNormal(seed * 2 + 2, sigma, target, (size_t)outChannels * inChannels * kernelDim.height * kernelDim.width);
}

struct options {
    size_t input_channels;
    size_t output_channels;
    struct nnp_size input_size;
    size_t input_padding;
    struct nnp_size kernel_size;
    struct nnp_size output_subsampling;
    enum nnp_convolution_algorithm algorithm;
    enum nnp_convolution_transform_strategy transform_strategy;
    enum nnp_convolution_tuning_strategy tuning_strategy;
    size_t threads;
    size_t iterations;
    size_t batch;
    uint64_t seed;
    bool blocked_variant;
    bool variant_given;
    bool check;
    size_t check_images;
    bool strict;
    bool json;
};

void print_options_help(const char *program_name) {
    printf(
        "%s parameters...\n"
        "Required parameters:\n"
        "  -ic  --input-channels     The number of input channels\n"
        "  -oc  --output-channels    The number of output channels\n"
        "  -is  --input-size         Input height and width\n"
        "  -ks  --kernel-size        Kernel height and width\n"
        "Optional parameters:\n"
        "  -a   --algorithm          The algorithm (auto, direct, im2col, or winograd) for computing convolution (default: auto)\n"
        "  -ts  --transform-strategy The transformation strategy (online, or offline) for kernel transformation (default: online)\n"
        "  -s   --output-subsampling The size of a output subsampling region, AKA stride (default: 1x1)\n"
        "  -ip  --input-padding      Implicit input padding (default: 1)\n"
        "  -tn  --tuning             whether to tuning (default: no_tuning)\n"
        "  -t   --threads            The number of host threads for the naive check (default: 1)\n"
        "  -i   --iterations         # iterations (default: 10)\n"
        "  -n   --batch              Images per forward pass (default: 1)\n"
        "       --seed               Seed of the input generator (default: 0)\n"
        "       --variant            Winograd pipeline: zc (four staged kernels) or blocked (no M buffer / single kernel);\n"
        "                            default: whichever the library prefers for the layer\n"
        "       --no-check           Skip the naive reference and the error check\n"
        "       --check-images       Check only the last K images of the batch against the naive reference\n"
        "                            (default: all; the host convolution of a large batch takes minutes)\n"
        "       --strict             Exit with status 2 when the error exceeds the tolerance\n"
        "       --json               Also print one JSON line with the results\n",
        program_name);
}

static bool is_flag(const char *arg, const char *long_name, const char *short_name) {
    return strcmp(arg, long_name) == 0 || (short_name && strcmp(arg, short_name) == 0);
}

static size_t parse_count(int argc, char **argv, int i, const char *what, bool allow_zero) {
    if (i + 1 >= argc) {
        fprintf(stderr, "Error: expected %s value\n", what);
        exit(EXIT_FAILURE);
    }
    size_t v = 0;
    if (argv[i + 1][0] == '-' || sscanf(argv[i + 1], "%zu", &v) != 1) {
        fprintf(stderr, "Error: can not parse %s as an unsigned integer\n", argv[i + 1]);
        exit(EXIT_FAILURE);
    }
    if (v == 0 && !allow_zero) {
        fprintf(stderr, "Error: invalid value %s for the %s: positive value expected\n", argv[i + 1], what);
        exit(EXIT_FAILURE);
    }
    return v;
}

static nnp_size parse_pair(int argc, char **argv, int i, const char *what) {
    if (argc - i < 2) {
        fprintf(stderr, "Error: expected two %s values\n", what);
        exit(EXIT_FAILURE);
    }
    nnp_size s;
    s.height = parse_count(argc, argv, i, what, false);
    s.width = parse_count(argc, argv, i + 1, what, false);
    return s;
}

struct options parse_options(int argc, char **argv) {
    struct options options;
    options.input_channels = 0;
    options.output_channels = 0;
    options.input_size = {0, 0};
    options.input_padding = 1;
    options.kernel_size = {0, 0};
    options.output_subsampling = {1, 1};
    options.algorithm = nnp_convolution_algorithm_auto;
    options.transform_strategy = nnp_convolution_transform_strategy_online;
    options.tuning_strategy = nnp_convolution_tuning_strategy_no_tuning;
    options.threads = 1;
    options.iterations = 10;
    options.batch = 1;
    options.seed = 0;
    options.blocked_variant = false;
    options.variant_given = false;
    options.check = true;
    options.check_images = 0;
    options.strict = false;
    options.json = false;

    for (int i = 1; i < argc; i += 1) {
        if (is_flag(argv[i], "--input-channels", "-ic")) {
            options.input_channels = parse_count(argc, argv, i, "number of input channels", false);
            i += 1;
        } else if (is_flag(argv[i], "--output-channels", "-oc")) {
            options.output_channels = parse_count(argc, argv, i, "number of output channels", false);
            i += 1;
        } else if (is_flag(argv[i], "--input-size", "-is")) {
            options.input_size = parse_pair(argc, argv, i, "input size");
            i += 2;
        } else if (is_flag(argv[i], "--kernel-size", "-ks")) {
            options.kernel_size = parse_pair(argc, argv, i, "kernel size");
            i += 2;
        } else if (is_flag(argv[i], "--input-padding", "-ip")) {
            options.input_padding = parse_count(argc, argv, i, "input padding", true);
            i += 1;
        } else if (is_flag(argv[i], "--output-subsampling", "-s")) {
            options.output_subsampling = parse_pair(argc, argv, i, "output subsampling");
            i += 2;
        } else if (is_flag(argv[i], "--algorithm", "-a")) {
            if (i + 1 == argc) {
                fprintf(stderr, "Error: expected convolution algorithm name\n");
                exit(EXIT_FAILURE);
            }
            if (strcmp(argv[i + 1], "auto") == 0) options.algorithm = nnp_convolution_algorithm_auto;
            else if (strcmp(argv[i + 1], "direct") == 0) options.algorithm = nnp_convolution_algorithm_direct;
            else if (strcmp(argv[i + 1], "im2col") == 0) options.algorithm = nnp_convolution_algorithm_im2col;
            else if (strcmp(argv[i + 1], "winograd") == 0) options.algorithm = nnp_convolution_algorithm_winograd;
            else {
                fprintf(stderr, "Error: invalid convolution algorithm name %s\n", argv[i + 1]);
                exit(EXIT_FAILURE);
            }
            i += 1;
        } else if (is_flag(argv[i], "--transform-strategy", "-ts")) {
            if (i + 1 == argc) {
                fprintf(stderr, "Error: expected transformation strategy name\n");
                exit(EXIT_FAILURE);
            }
            if (strcmp(argv[i + 1], "online") == 0) options.transform_strategy = nnp_convolution_transform_strategy_online;
            else if (strcmp(argv[i + 1], "offline") == 0) options.transform_strategy = nnp_convolution_transform_strategy_offline;
            else {
                fprintf(stderr, "Error: invalid transformation strategy name %s\n", argv[i + 1]);
                exit(EXIT_FAILURE);
            }
            i += 1;
        } else if (is_flag(argv[i], "--tuning", "-tn")) {
            if (i + 1 == argc) {
                fprintf(stderr, "Error: expected tuning strategy name\n");
                exit(EXIT_FAILURE);
            }
            if (strcmp(argv[i + 1], "no_tuning") == 0) options.tuning_strategy = nnp_convolution_tuning_strategy_no_tuning;
            else if (strcmp(argv[i + 1], "tuning") == 0) options.tuning_strategy = nnp_convolution_tuning_strategy_grid_search;
            else {
                fprintf(stderr, "Error: invalid tuning strategy name %s\n", argv[i + 1]);
                exit(EXIT_FAILURE);
            }
            i += 1;
        } else if (is_flag(argv[i], "--threads", "-t")) {
            options.threads = parse_count(argc, argv, i, "number of threads", false);
            i += 1;
        } else if (is_flag(argv[i], "--iterations", "-i")) {
            options.iterations = parse_count(argc, argv, i, "number of iterations", false);
            i += 1;
        } else if (is_flag(argv[i], "--batch", "-n")) {
            options.batch = parse_count(argc, argv, i, "batch size", false);
            i += 1;
        } else if (is_flag(argv[i], "--seed", NULL)) {
            options.seed = parse_count(argc, argv, i, "seed", true);
            i += 1;
        } else if (is_flag(argv[i], "--variant", NULL)) {
            if (i + 1 == argc || (strcmp(argv[i + 1], "zc") != 0 && strcmp(argv[i + 1], "blocked") != 0)) {
                fprintf(stderr, "Error: expected winograd variant zc or blocked\n");
                exit(EXIT_FAILURE);
            }
            options.blocked_variant = strcmp(argv[i + 1], "blocked") == 0;
            options.variant_given = true;
            i += 1;
        } else if (is_flag(argv[i], "--no-check", NULL)) {
            options.check = false;
        } else if (is_flag(argv[i], "--check-images", NULL)) {
            options.check_images = parse_count(argc, argv, i, "number of checked images", false);
            i += 1;
        } else if (is_flag(argv[i], "--strict", NULL)) {
            options.strict = true;
        } else if (is_flag(argv[i], "--json", NULL)) {
            options.json = true;
        } else if (is_flag(argv[i], "--help", "-h")) {
            print_options_help(argv[0]);
            exit(EXIT_SUCCESS);
        } else {
            fprintf(stderr, "Error: unknown argument '%s'\n", argv[i]);
            print_options_help(argv[0]);
            exit(EXIT_FAILURE);
        }
    }
    if (options.input_channels == 0) {
        fprintf(stderr, "Error: the number of input channels is not specified\n");
        print_options_help(argv[0]);
        exit(EXIT_FAILURE);
    }
    if (options.output_channels == 0) {
        fprintf(stderr, "Error: the number of output channels is not specified\n");
        print_options_help(argv[0]);
        exit(EXIT_FAILURE);
    }
    if (options.input_size.width == 0) {
        fprintf(stderr, "Error: the input size is not specified\n");
        print_options_help(argv[0]);
        exit(EXIT_FAILURE);
    }
    if (options.kernel_size.width == 0) {
        fprintf(stderr, "Error: the kernel size is not specified\n");
        print_options_help(argv[0]);
        exit(EXIT_FAILURE);
    }
    return options;
}

static const char *algorithm_name(enum nnp_convolution_algorithm a) {
    switch (a) {
        case nnp_convolution_algorithm_direct: return "direct";
        case nnp_convolution_algorithm_im2col: return "im2col";
        case nnp_convolution_algorithm_winograd: return "winograd";
        default: return "auto";
    }
}

int main(int argc, char *argv[]) {
    struct options options = parse_options(argc, argv);

    const size_t input_channels = options.input_channels;
    const size_t output_channels = options.output_channels;
    const struct nnp_padding input_padding = {options.input_padding, options.input_padding, options.input_padding,
                                              options.input_padding};
    const struct nnp_size input_size = options.input_size;
    const struct nnp_size kernel_size = options.kernel_size;
    const struct nnp_size output_subsampling = options.output_subsampling;
    if (input_padding.left + input_size.width + input_padding.right < kernel_size.width ||
        input_padding.top + input_size.height + input_padding.bottom < kernel_size.height) {
        fprintf(stderr, "Error: the kernel is larger than the padded input\n");
        exit(EXIT_FAILURE);
    }
    const struct nnp_size output_size = {
        (input_padding.left + input_size.width + input_padding.right - kernel_size.width) / output_subsampling.width + 1,
        (input_padding.top + input_size.height + input_padding.bottom - kernel_size.height) / output_subsampling.height + 1};

    printf("Batch: %zu\n", options.batch);
    printf("Input channels: %zu\n", input_channels);
    printf("Output channels: %zu\n", output_channels);
    printf("Input: %zux%zu with implicit padding %zu\n", input_size.height, input_size.width, options.input_padding);
    printf("Kernel: %zux%zu\n", kernel_size.height, kernel_size.width);
    printf("Subsampling: %zux%zu\n", output_subsampling.height, output_subsampling.width);

    const size_t in_elems = options.batch * input_size.height * input_size.width * input_channels;
    const size_t k_elems = kernel_size.height * kernel_size.width * input_channels * output_channels;
    const size_t out_elems = options.batch * output_channels * output_size.height * output_size.width;
    float *test_input = (float *)malloc(sizeof(float) * in_elems);
    float *test_kernel = (float *)malloc(sizeof(float) * k_elems);
    if (!test_input || !test_kernel) {
        fprintf(stderr, "Buffer is NULL.\n");
        exit(EXIT_FAILURE);
    }
    fillTestInput(test_input, options.batch, (int)input_channels, input_size, options.seed);
    fillTestKernel(test_kernel, (int)input_channels, (int)output_channels, kernel_size, options.seed);

    // the naive reference covers the whole batch, or its last --check-images images
    const size_t checked = (options.check_images && options.check_images < options.batch) ? options.check_images : options.batch;
    const size_t first_checked = options.batch - checked;
    const bool partial_check = checked < options.batch;
    ConvNaiveLayer *conv_reference = NULL;
    double naive_ms = 0.0;
    if (options.check) {
        conv_reference = new ConvNaiveLayer(test_input + first_checked * (in_elems / options.batch), test_kernel, NULL, NULL,
                                            input_channels, input_size.height,
                                            input_size.width, output_channels, kernel_size.height, kernel_size.width,
                                            output_subsampling.height, output_subsampling.width, input_padding.left,
                                            input_padding.right, input_padding.top, input_padding.bottom, 1, false,
                                            options.threads, 1, checked);
        Timer naive;
        naive.startBench();
        conv_reference->Forward();
        naive_ms = naive.endBench(1.0);
        printf("Naive reference on %zu host thread(s), %zu of %zu image(s): %.3f ms\n", options.threads, checked,
               options.batch, naive_ms);
    }
    float *output_ref = conv_reference ? conv_reference->output_data : NULL;
    // the layers compare their whole output with the array they are given (the reference's diff()):
    // with a partial reference that comparison is made here instead
    float *layer_ref = partial_check ? NULL : output_ref;

    if (options.algorithm == nnp_convolution_algorithm_auto)
        options.algorithm = select_algorithm(kernel_size, output_subsampling, output_size, input_channels,
                                             output_channels, options.batch);
    if (options.algorithm == nnp_convolution_algorithm_winograd &&
        (kernel_size.height != 3 || kernel_size.width != 3 || output_subsampling.height != 1 ||
         output_subsampling.width != 1)) {
        fprintf(stderr, "Error: winograd supports only 3x3 kernels with stride 1\n");
        exit(EXIT_FAILURE);
    }
    printf("Selected algorithm: %s\n", algorithm_name(options.algorithm));

    // arena: input, filter, output, plus the algorithm's scratch (U, V, M are 64 planes each)
    {
        const size_t tiles = options.batch * ((output_size.height + 5) / 6) * ((output_size.width + 5) / 6);
        const size_t cpad = (input_channels + 31) / 32 * 32, kpad = (output_channels + 255) / 256 * 256;
        const size_t tpad = (tiles + 255) / 256 * 256;
        size_t bytes = 4 * (in_elems + 2 * k_elems + out_elems) + ((size_t)64 << 20);
        if (options.algorithm == nnp_convolution_algorithm_winograd)
            bytes += 4 * 64 * (cpad * kpad + cpad * tpad + kpad * tpad);
        else
            bytes += 4 * ((k_elems / output_channels + 32) * kpad) + 8 * (k_elems / output_channels + 32) +
                     std::min<size_t>(32 * 4 * out_elems, (size_t)1 << 30);   // split-reduction workspace of small layers
        fastconv::Device::Configure(bytes);
    }

    ConvLayer *conv_test = NULL;
    double tolerance = 1e-5;
    int chosen_config = -1;
    int chosen_option = -1;                 // blocked Winograd: images per block (0 = single-kernel engine)
    int kernel_transform_offline = -1;      // Winograd: 1 = filter transformed once in Init(), 0 = in every pass
    double stage_ms[4] = {0, 0, 0, 0};
    switch (options.algorithm) {
        case nnp_convolution_algorithm_auto:
            break;
        case nnp_convolution_algorithm_direct:
        case nnp_convolution_algorithm_im2col: {
            // "direct" (1x1 stride 1) is the same kernel: with a 1x1 window the gather is a plain row read
            ConvIm2colLayer *conv = new ConvIm2colLayer(
                test_input, test_kernel, NULL, layer_ref, input_channels, input_size.height, input_size.width,
                output_channels, kernel_size.height, kernel_size.width, output_subsampling.height,
                output_subsampling.width, input_padding.left, input_padding.right, input_padding.top,
                input_padding.bottom, 1, false, options.threads, options.iterations, options.batch);
            if (options.tuning_strategy != nnp_convolution_tuning_strategy_no_tuning) conv->Tuning();
            conv->Init();
            conv->Forward();
            chosen_config = conv->best_config();
            stage_ms[2] = conv->gemm_ms;
            conv_test = conv;
        } break;
        case nnp_convolution_algorithm_winograd: {
            tolerance = 1e-3;
            if (!options.variant_given) {
                // few-channel layers are faster without V and M round trips through HBM
                fc_conv_shape shp = {(int)options.batch, (int)input_channels, (int)input_size.height, (int)input_size.width,
                                     (int)output_channels, 3, 3, 1, 1, (int)input_padding.top, (int)input_padding.bottom,
                                     (int)input_padding.left, (int)input_padding.right};
                options.blocked_variant = fc_wino_prefer_onepass(&shp) || fc_wino_prefer_fused(&shp);
            }
            if (options.blocked_variant) {
                ConvWinoF63Layer *conv = new ConvWinoF63Layer(
                    test_input, test_kernel, NULL, layer_ref, input_channels, input_size.height, input_size.width,
                    output_channels, kernel_size.height, kernel_size.width, output_subsampling.height,
                    output_subsampling.width, input_padding.left, input_padding.right, input_padding.top,
                    input_padding.bottom, 1, false, options.threads, options.iterations, options.batch);
                if (options.tuning_strategy != nnp_convolution_tuning_strategy_no_tuning) conv->Tuning();
                else conv->SetOfflineKernelTransform(options.transform_strategy == nnp_convolution_transform_strategy_offline);
                conv->Init();
                conv->Forward();
                chosen_config = conv->best_config();
                chosen_option = conv->best_images_per_block();
                kernel_transform_offline = conv->best_offline();
                for (int i = 0; i < 4; i++) stage_ms[i] = conv->stage_ms[i];
                conv_test = conv;
            } else {
                ConvWinoF63ZCLayer *conv = new ConvWinoF63ZCLayer(
                    test_input, test_kernel, NULL, layer_ref, input_channels, input_size.height, input_size.width,
                    output_channels, kernel_size.height, kernel_size.width, output_subsampling.height,
                    output_subsampling.width, input_padding.left, input_padding.right, input_padding.top,
                    input_padding.bottom, 1, false, options.threads, options.iterations, options.batch);
                if (options.tuning_strategy != nnp_convolution_tuning_strategy_no_tuning)
                    conv->Tuning();
                else if (options.transform_strategy == nnp_convolution_transform_strategy_offline)
                    conv->SetConfig(conv->best_config(), 1);
                conv->Init();
                conv->Forward();
                chosen_config = conv->best_config();
                kernel_transform_offline = conv->best_offline();
                for (int i = 0; i < 4; i++) stage_ms[i] = conv->stage_ms[i];
                conv_test = conv;
            }
        } break;
    }

    int status = 0;
    if (conv_test) {
        const double ms = conv_test->last_total_ms;
        const double gflops = conv_test->flops() / (ms * 1e-3) / 1e9;
        printf("Effective GFLOP/s: %.1f (direct-convolution FLOP count %.3f GFLOP, %.4f ms per forward)\n", gflops,
               conv_test->flops() / 1e9, ms);
        double err = -1.0;
        if (output_ref) {
            const size_t out_img = out_elems / options.batch;
            err = max_rel_err(conv_test->output_data + first_checked * out_img, output_ref, checked * out_img);
            const bool ok = err <= tolerance;
            printf("Max relative error vs naive: %.3e (tolerance %.0e) %s\n", err, tolerance, ok ? "PASS" : "FAIL");
            if (!ok && options.strict) status = 2;
        }
        if (options.json) {
            // Each stage against the roofline that bounds it (MI355X: 157.3 TFLOP/s of fp32 MFMA, 8 TB/s of HBM),
            // from the algorithmic work of the stage: Winograd products 2*64*K*C*T flop over T = N*ceil(OH/6)*ceil(OW/6)
            // tiles (the implicit GEMM: the direct-convolution count), input transform x once + V once, output
            // transform M once + y once, filter transform w once + U once.
            const double kPeakTflops = 157.3, kPeakGbs = 8000.0;
            const bool wino = options.algorithm == nnp_convolution_algorithm_winograd;
            const double N = (double)options.batch, C = (double)input_channels, K = (double)output_channels;
            const double T = N * (double)((output_size.height + 5) / 6) * (double)((output_size.width + 5) / 6);
            const double gemm_flops = wino ? 2.0 * 64.0 * K * C * T : conv_test->flops();
            const double it_bytes = 4.0 * N * C * (double)input_size.height * (double)input_size.width + 256.0 * C * T;
            const double ot_bytes = 256.0 * K * T + 4.0 * N * K * (double)output_size.height * (double)output_size.width;
            const double kt_bytes = 4.0 * K * C * (9.0 + 64.0);
            char roof[512];
            int at = 0;
            auto field = [&](const char *name, double work, double stage, double unit, double peak, const char *frac_name) {
                if (stage > 0.0) {
                    const double rate = work / (stage * 1e-3) / unit;
                    at += snprintf(roof + at, sizeof roof - at, ", \"%s\": %.2f, \"%s\": %.4f", name, rate, frac_name, rate / peak);
                } else {
                    at += snprintf(roof + at, sizeof roof - at, ", \"%s\": null, \"%s\": null", name, frac_name);
                }
            };
            field("gemm_tflops", gemm_flops, stage_ms[2], 1e12, kPeakTflops, "gemm_frac_mfma");
            field("input_tran_gbs", it_bytes, wino ? stage_ms[0] : 0.0, 1e9, kPeakGbs, "input_tran_frac_hbm");
            field("output_tran_gbs", ot_bytes, wino ? stage_ms[3] : 0.0, 1e9, kPeakGbs, "output_tran_frac_hbm");
            field("kernel_tran_gbs", kt_bytes, wino ? stage_ms[1] : 0.0, 1e9, kPeakGbs, "kernel_tran_frac_hbm");
            printf("{\"algorithm\": \"%s%s\", \"batch\": %zu, \"ic\": %zu, \"oc\": %zu, \"ih\": %zu, \"iw\": %zu, "
                   "\"kh\": %zu, \"kw\": %zu, \"stride\": %zu, \"pad\": %zu, \"config\": %d, \"ms\": %.6f, "
                   "\"gflops\": %.2f, \"input_tran_ms\": %.6f, \"kernel_tran_ms\": %.6f, \"gemm_ms\": %.6f, "
                   "\"output_tran_ms\": %.6f, \"max_rel_err\": %.4e, \"naive_ms\": %.3f, \"naive_threads\": %zu, "
                   "\"checked_images\": %zu, \"images_per_block\": %d, \"kernel_transform\": \"%s\"%s, "
                   "\"peak_mfma_tflops\": %.1f, \"peak_hbm_gbs\": %.0f}\n",
                   algorithm_name(options.algorithm),
                   (options.algorithm == nnp_convolution_algorithm_winograd && options.blocked_variant) ? "_blocked" : "",
                   options.batch, input_channels, output_channels, input_size.height, input_size.width,
                   kernel_size.height, kernel_size.width, output_subsampling.height, options.input_padding,
                   chosen_config, ms, gflops, stage_ms[0], stage_ms[1], stage_ms[2], stage_ms[3], err, naive_ms,
                   options.threads, options.check ? checked : (size_t)0, chosen_option,
                   kernel_transform_offline < 0 ? "n/a" : kernel_transform_offline ? "offline" : "online", roof,
                   kPeakTflops, kPeakGbs);
        }
    }
    delete conv_test;
    delete conv_reference;
    free(test_input);
    free(test_kernel);
    return status;
}
