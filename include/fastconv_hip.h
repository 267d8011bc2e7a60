/*
 * fastconv_hip.h -- C ABI of the MI355X (gfx950) convolution kernels.
 *
 * This is the boundary the C++ host layers (ConvWinoF63ZCLayer, ConvWinoF63Layer,
 * ConvIm2colLayer) call; it is also what any other binding (ctypes, cgo, JNI)
 * would load.  Plain pointers and sizes only.  Every function returns 0
 * (FC_OK) or a negative fc_status; nothing throws across the boundary.  A
 * context owns one HIP stream; calls on one context are ordered on that stream
 * and must come from one thread at a time.
 *
 * Each entry point names the reference interface it stands in for (paths
 * relative to the reference checkout).
 */
#ifndef FASTCONV_HIP_H_
#define FASTCONV_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    FC_OK = 0,
    FC_ERR_INVALID = -1,      /* bad argument / unsupported shape for this entry point */
    FC_ERR_NO_DEVICE = -2,    /* no usable gfx950 device */
    FC_ERR_HIP = -3,          /* a HIP runtime call failed; see fc_last_error() */
    FC_ERR_OOM = -4,          /* pool exhausted or hipMalloc failed */
    FC_ERR_STATE = -5,        /* call made in the wrong order (e.g. after destroy) */
    FC_ERR_UNSUPPORTED = -6   /* size beyond a stated limit of the kernel */
} fc_status;

typedef struct fc_context fc_context;
typedef struct fc_pool fc_pool;

/* Convolution geometry, fp32 NCHW, group 1.  Field meaning follows the
 * ConvLayer constructor arguments (conv_layer.h:27) plus a batch count. */
typedef struct {
    int N, C, H, W;
    int K, kh, kw;
    int sh, sw;
    int pt, pb, pl, pr;
} fc_conv_shape;

/* Stages whose device time can be read back, labelled as the reference prints
 * them (convLayer/winoF63ConvZC.cpp:249-253, convLayer/im2colConv.cpp:254-256). */
typedef enum {
    FC_STAGE_KERNEL_TRAN = 0,
    FC_STAGE_INPUT_TRAN = 1,
    FC_STAGE_TENSOR_GEMM = 2,
    FC_STAGE_OUTPUT_TRAN = 3,
    FC_STAGE_IMPLICIT_GEMM = 4,
    FC_STAGE_FILTER_PACK = 5,
    FC_STAGE_FUSED_GEMM_OUT = 6,
    FC_STAGE_ONEPASS = 7,
    FC_STAGE_COUNT = 8
} fc_stage;

typedef struct {
    char name[128];
    char arch[32];
    int compute_units;
    int clock_mhz;
    int mem_clock_mhz;
    int mem_bus_bits;
    size_t total_mem;
    int lds_per_block;
} fc_device_info;

/* ---- context ---------------------------------------------------------- */

/* Replaces the implicit process-wide state of the reference (one process,
 * OpenMP threads set in conv_layer.h:31).  Fails with FC_ERR_NO_DEVICE when no
 * GPU is present: there is no CPU fallback. */
int fc_init(int device, fc_context **out);
int fc_destroy(fc_context *ctx);
int fc_get_device_info(fc_context *ctx, fc_device_info *info);
const char *fc_last_error(fc_context *ctx);
const char *fc_status_string(int status);
int fc_sync(fc_context *ctx);

/* ---- memory: one hipMalloc'd arena ------------------------------------ */

/* Stands in for the allocations behind CommonMemPool / PrivateMemPool
 * (utility/mempool.h:23-71) and _mm_malloc (utility/common.cpp:26-40): one
 * device allocation per pool, sub-allocated by bumping a 256-byte aligned
 * offset.  fc_pool_reset() rewinds to empty; fc_pool_mark/release rewind to a
 * saved offset (scratch that lives for one Tuning() candidate). */
int fc_pool_create(fc_context *ctx, size_t bytes, fc_pool **out);
int fc_pool_destroy(fc_pool *pool);
int fc_pool_alloc(fc_pool *pool, size_t bytes, void **dev_ptr);
int fc_pool_reset(fc_pool *pool);
int fc_pool_mark(fc_pool *pool, size_t *mark);
int fc_pool_release(fc_pool *pool, size_t mark);
int fc_pool_stats(fc_pool *pool, size_t *capacity, size_t *used, size_t *peak);

/* Stand in for the memcpy()s into the layer's own buffers (conv_layer.h:74-77). */
int fc_upload(fc_context *ctx, void *dst_dev, const void *src_host, size_t bytes);
int fc_download(fc_context *ctx, void *dst_host, const void *src_dev, size_t bytes);
int fc_fill_zero(fc_context *ctx, void *dst_dev, size_t bytes);
/* Device-to-device copy by a plain kernel (16 bytes per lane): the known-size
 * reference that hardware traffic counters are scaled by.  Both pointers and the
 * size must be multiples of 16. */
int fc_device_copy(fc_context *ctx, void *dst_dev, const void *src_dev, size_t bytes);

/* Synthetic inputs of the drivers, written to HOST memory: n floats uniform in [lo, hi), or
 * normal with standard deviation sigma (Box-Muller in double), from a splitmix64-seeded
 * xoshiro256** stream, so that every machine sees the same layer for a given seed.  Stand in
 * for fillTestInput / fillTestKernel (ConvTest.cpp:18-46), which draw from rand(). */
int fc_host_fill_uniform(uint64_t seed, float lo, float hi, float *dst_host, size_t n);
int fc_host_fill_normal(uint64_t seed, float sigma, float *dst_host, size_t n);

/* ---- stage timing (utility/helper.h:66-80 Timer, per stage) ----------- */

/* stage_mask has bit (1 << stage) set for every stage whose kernel launches are
 * to be bracketed by two events on the context's stream (FC_TIMING_ALL for all,
 * 0 to switch timing off).  fc_stage_time_ms() waits for the stream, folds the
 * pending event pairs into per-stage totals and returns total milliseconds and
 * launch count since the last fc_timing_reset(). */
#define FC_TIMING_ALL 0xff
int fc_timing_enable(fc_context *ctx, int stage_mask);
int fc_timing_reset(fc_context *ctx);
int fc_stage_time_ms(fc_context *ctx, int stage, double *total_ms, long *launches);

/* Shader clock under load.  The published MFMA peak is quoted at the maximum shader clock
 * (2400 MHz on MI355X); under fp32 MFMA load with real data the chip's power management runs
 * the shaders slower, and the clock it sustains is what bounds the products.
 * fc_clock_probe_begin starts a one-wavefront kernel on a stream of its own that, `samples`
 * times (1..256), waits `sample_us` microseconds (1..100000) on the constant 100 MHz counter and
 * records how far the shader-clock counter moved meanwhile; work enqueued through this context
 * afterwards runs beside it.  fc_clock_probe_end waits for the probe and returns the shader
 * clock of every sample in MHz (at most `capacity` of them; *n_samples = how many were taken).
 * One probe at a time per context; not while a graph is being recorded.  No counterpart in the
 * reference, whose Timer (utility/helper.cpp:113-148) sees wall time only. */
int fc_clock_probe_begin(fc_context *ctx, int samples, int sample_us);
int fc_clock_probe_end(fc_context *ctx, double *mhz, int capacity, int *n_samples);

/* ---- Winograd F(6x6,3x3), stride 1 ------------------------------------ */

/* Tile shapes of the batched GEMM stage.  The reference tunes
 * ocBlock/tileBlock/icBlock and a 4x4 or 4x5 register kernel
 * (convLayer/winoF63ConvZC.cpp:25-174); here a configuration is a workgroup
 * tile BM (output channels) x BN (tiles) x BK (input channels) and a wave grid
 * (waves_m x waves_n wavefronts side by side over the tile, times waves_k
 * wavefronts that each take a share of the reduction). */
typedef struct {
    int id;
    int bm, bn, bk;
    int waves_m, waves_n;
    int lds_bytes;
    int waves_k;              /* wavefronts of a workgroup that split the reduction among themselves (1: no split) */
} fc_gemm_config;

int fc_wino_gemm_num_configs(void);
int fc_wino_gemm_get_config(int id, fc_gemm_config *cfg);
/* Tile shape to use when a layer has not been tuned (the role of the defaults
 * ocBlock=140, tileBlock=52, icBlock=64 in convLayer/winoF63ConvZC.cpp:11-16):
 * the shape with the least padded work, discounted for narrow tiles and for
 * grids that leave compute units idle.  Returns a configuration id. */
int fc_wino_gemm_default_config(const fc_conv_shape *shape);

/* Buffer geometry for one layer under one GEMM configuration.  Frequencies
 * f = 8*row + col of the transformed 8x8 tile; tiles t = (n*tiles_h + th)*tiles_w + tw.
 *   U[64][C_pad][K_pad]   transformed filters, output channel fastest
 *   V[64][C_pad][T_pad]   transformed input tiles, tile fastest
 *   M[64][K_pad][T_pad]   per-frequency products, tile fastest
 * Padding (to the GEMM tile) is written as zeros by the transforms.
 * Stands in for the buffer sizing in ConvWinoF63ZCLayer::Init
 * (convLayer/winoF63ConvZC.cpp:176-213). */
typedef struct {
    fc_conv_shape shape;
    int OH, OW;
    int tiles_h, tiles_w;
    long T;
    int K_pad, C_pad;
    long T_pad;
    int gemm_config;
    size_t U_bytes, V_bytes, M_bytes;
} fc_wino_plan;

/* FC_ERR_INVALID unless the layer is 3x3 with stride 1; FC_ERR_UNSUPPORTED when the output is
 * wider than 1020 columns (170 tiles: two bands of the input transform must fit 64 KiB of LDS)
 * or a buffer would pass 2^31 elements per frequency plane.  Every later call checks the plan it
 * is given against the one this function makes for plan->shape and plan->gemm_config. */
int fc_wino_make_plan(const fc_conv_shape *shape, int gemm_config, fc_wino_plan *plan);

/* The rule behind `-a auto` for one layer (select_algorithm, ConvTest.cpp:318-331, which looks at
 * filter size and stride only): 1 when the Winograd path is expected to be faster than the
 * implicit GEMM on MI355X, 0 when not or when Winograd cannot run the layer at all (not 3x3
 * stride 1, or wider than fc_wino_make_plan admits).  The thresholds come from measured
 * per-layer times of both paths on the VGG-16 and ResNet-50 layers at batch 1 and 32. */
int fc_prefer_winograd(const fc_conv_shape *shape);

/* U = G g G^T.  Replaces the kernel transform inside winoF63_v1_single
 * (winoF63ZC/winoF63ZC.cpp:433-500) and offline_kernel_transform_v1 (:242-322).
 * w is K x C x 3 x 3. */
int fc_wino_filter_transform(fc_context *ctx, const fc_wino_plan *plan,
                             const float *w_dev, float *U_dev);

/* V = B^T d B with zero-filled borders.  Replaces the input transform inside
 * winoF63_v1_single (winoF63ZC/winoF63ZC.cpp:512-813). */
int fc_wino_input_transform(fc_context *ctx, const fc_wino_plan *plan,
                            const float *x_dev, float *V_dev);

/* Both transforms above in one launch (the filter transform of a layer is a short kernel;
 * launched by itself it costs a launch and a drain of the chip per layer).  What the online
 * strategy of winoF63_v1_single does back to back (winoF63ZC/winoF63ZC.cpp:433-813).  Its
 * time is booked under FC_STAGE_INPUT_TRAN. */
int fc_wino_filter_input_transform(fc_context *ctx, const fc_wino_plan *plan,
                                   const float *w_dev, float *U_dev,
                                   const float *x_dev, float *V_dev);

/* M[f] = U[f]^T-layout product over input channels for all 64 frequencies in
 * one launch, on fp32 MFMA.  Replaces the depth x oc x tile loop nest calling
 * TensorGEMMInnerKernel4x4x4_v3 (winoF63ZC/winoF63ZC.cpp:818-860,
 * winoF63ZC/TensorGEMMZC.cpp:443-583).  M is overwritten, never accumulated. */
int fc_wino_gemm(fc_context *ctx, const fc_wino_plan *plan,
                 const float *U_dev, const float *V_dev, float *M_dev);

/* The same stage fed by the untransformed filter w[K][C][3][3]: U = G g G^T is formed
 * in registers, lane by lane in the layout the MFMA takes its first operand in, and never
 * exists in memory.  For layers with few tiles (batch 1 on 7x7 to 28x28 images), where
 * the stage above is one pass over U, 64/9 times the size of w.  Like the reference's
 * online strategy (kernel transform inside Forward, ConvTest.cpp:230-243) without its
 * kernelBuf.  Needs plan->T <= 64 and C a multiple of 16
 * (fc_wino_raw_filter_gemm_applies); freqs_per_wave = 0 lets the library choose how many
 * of the 64 frequencies a wavefront multiplies (1, 2 or 4) and channel_split = 0 over how
 * many groups of wavefronts a workgroup spreads the input channels (1, 2 or 4): tuning
 * parameters like the tile shape of fc_wino_gemm.  M is overwritten: rows K up to K rounded
 * up to 16 are written as zeros and columns T up to T rounded up to 16, 32 or 64 hold the
 * products of V's (zero) padding; rows and columns beyond that, up to K_pad and T_pad, are
 * left as they were.  The output transform reads none of the padding. */
int fc_wino_gemm_raw_filter(fc_context *ctx, const fc_wino_plan *plan,
                            const float *w_dev, const float *V_dev, float *M_dev,
                            int freqs_per_wave, int channel_split);
int fc_wino_raw_filter_gemm_applies(const fc_wino_plan *plan);
/* 1 when fc_wino_gemm_raw_filter is expected to beat filter transform + fc_wino_gemm
 * (measured on MI355X: at most 32 tiles and C*K >= 32768).  Against fc_wino_gemm alone,
 * with the filter transformed beforehand, the two are level. */
int fc_wino_prefer_raw_filter_gemm(const fc_wino_plan *plan);

/* Y = A^T m A clipped to the image, written NCHW, with an optional per-channel
 * bias (K floats) and optional ReLU.  Replaces the output transform inside
 * winoF63_v1_single (winoF63ZC/winoF63ZC.cpp:869-973). */
int fc_wino_output_transform(fc_context *ctx, const fc_wino_plan *plan,
                             const float *M_dev, const float *bias_dev, int relu,
                             float *y_dev);

/* GEMM and output transform in one kernel: the 64 per-frequency products of a
 * block of (32 output channels x 32 tiles) stay in registers and LDS, M is never
 * written (M_dev is not needed).  The counterpart of the reference's blocked
 * pipeline, where the GEMM result of one block is consumed by the output
 * transform out of block-local scratch (winoF63/winoF63.cpp:1574-1737).  Pays
 * when the transformed filter fits in L2 (C*K up to about 8192); any plan whose
 * C_pad is a multiple of 8 is accepted. */
int fc_wino_gemm_output_fused(fc_context *ctx, const fc_wino_plan *plan,
                              const float *U_dev, const float *V_dev,
                              const float *bias_dev, int relu, float *y_dev);

/* 1 when the fused kernel is expected to beat fc_wino_gemm + fc_wino_output_transform
 * for this layer (measured on MI355X: when the transformed filter, 256*C*K bytes,
 * stays L2-resident, C*K <= 8192, and the layer brings at least 512 blocks of 32 tiles x 32
 * output channels or has at most 8 input channels), else 0. */
int fc_wino_prefer_fused(const fc_conv_shape *shape);

/* Filter transform (unless filter_ready), input transform, fused GEMM + output
 * transform: the whole layer without an M buffer. */
int fc_wino_forward_fused(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                          const float *w_dev, const float *bias_dev, int relu, int filter_ready,
                          float *U_dev, float *V_dev, float *y_dev);

/* ---- the whole layer in one kernel ------------------------------------ */

/* gemm_config value of a plan made by fc_wino_make_onepass_plan. */
#define FC_WINO_ONEPASS (-1)

/* Plan for the single-kernel path: input transform, the 64 products and the output
 * transform inside one workgroup per (16 tiles x 64 output channels), so neither V nor M
 * exists (V_bytes = M_bytes = 0).  K_pad is K rounded up to 64, C_pad is C rounded up to 8.
 * The transformed filter uses its own layout, U4[64][C_pad/4][K_pad/64][4][16][4] (channel
 * 4q + c, output channel 64kb + 16sb + k at [f][q][kb][c][k][sb]); only
 * fc_wino_onepass_filter_transform writes it and
 * only fc_wino_conv_onepass reads it.  The stage calls above reject such a plan.
 * Images narrower than 8 columns are not supported (FC_ERR_UNSUPPORTED): use the staged calls.
 * Layers with at most four input channels (and an input of at most 2 GiB) run through a kernel
 * of their own on the vector ALUs behind the same three calls (the products are too few for the
 * matrix cores to matter and the layer is bound by the stores of y); their transformed filter
 * is laid out [K_pad][8][8][4] in the same buffer.
 * The GPU reading of the reference's blocked pipeline taken to its end: there one block of
 * tiles goes through input transform, TensorGEMM and output transform out of block-local
 * scratch (winoF63/winoF63.cpp:1574-1737); here the block-local scratch is LDS and registers. */
int fc_wino_make_onepass_plan(const fc_conv_shape *shape, fc_wino_plan *plan);

/* U4 = G g G^T in the layout above (offlineKernelTransform, winoF63/winoF63.cpp:846-973). */
int fc_wino_onepass_filter_transform(fc_context *ctx, const fc_wino_plan *plan,
                                     const float *w_dev, float *U_dev);

/* y = conv(x) (+bias, ReLU) from x and U4 in one launch. */
int fc_wino_conv_onepass(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                         const float *U_dev, const float *bias_dev, int relu, float *y_dev);

/* Filter transform (unless filter_ready) + fc_wino_conv_onepass.  U_dev holds the transformed filter
 * afterwards either way; for a layer with at most four input channels and few tiles the two run as one
 * launch (the convolution kernel transforms the filter itself and writes U_dev as a by-product, equal to
 * fc_wino_onepass_filter_transform's to the last bit or two). */
int fc_wino_forward_onepass(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                            const float *w_dev, const float *bias_dev, int relu, int filter_ready,
                            float *U_dev, float *y_dev);

/* 1 when the single-kernel path is expected to be the fastest Winograd pipeline for this
 * layer (measured on MI355X: 16 to 64 input channels, where the products are cheap next to
 * moving V and M through HBM, the image at least 8 columns wide, and at least 512 blocks of
 * 16 tiles x 64 output channels -- 192 when one block covers all output channels -- i.e. not
 * at batch 1; and every layer with at most four input channels, at any batch). */
int fc_wino_prefer_onepass(const fc_conv_shape *shape);

/* All stages back to back: what winoF63_v1_single (winoF63ZC/winoF63ZC.h:5-6)
 * does in one call.  filter_ready != 0 skips the filter transform (U already
 * holds it: the "offline" strategy, ConvTest.cpp:230-243).  With filter_ready == 0
 * the contents of U after the call are unspecified: a layer with few tiles
 * (fc_wino_prefer_raw_filter_gemm) multiplies straight from w and leaves U alone. */
int fc_wino_forward(fc_context *ctx, const fc_wino_plan *plan, const float *x_dev,
                    const float *w_dev, const float *bias_dev, int relu, int filter_ready,
                    float *U_dev, float *V_dev, float *M_dev, float *y_dev);

/* ---- implicit GEMM (replaces im2col + pack + GEMM) -------------------- */

int fc_igemm_num_configs(void);
int fc_igemm_get_config(int id, fc_gemm_config *cfg);
/* Untuned choice, as above (the role of mc=8, nc=256, kc=384 in
 * convLayer/im2colConv.h:17-18). */
int fc_igemm_default_config(const fc_conv_shape *shape);

/* Filter re-layout done once at Init: Wp[Kred_pad][K_pad], output channel
 * fastest, plus the per-row gather table.  The order of the reduction rows is
 * the library's business and depends on plan->config: the column matrix's
 * (c, r, s) (convLayer/im2colConv.cpp:285-309) in general, tap-major (r, s, c)
 * when C is a whole number of the configuration's reduction stages.  Treat Wp
 * and the table as opaque, hand them only to calls made with the same plan, and
 * pack them again when the configuration changes. */
typedef struct {
    fc_conv_shape shape;
    int OH, OW;
    int Kred, Kred_pad, K_pad;
    long Npix;
    int config;
    size_t Wp_bytes, table_bytes;
    int split_k;              /* > 1: the reduction is split over this many workgroups per tile */
    size_t ws_bytes;          /* workspace for the partial sums ([split_k][K][Npix] floats), 0 if unsplit */
} fc_igemm_plan;

int fc_igemm_make_plan(const fc_conv_shape *shape, int config, fc_igemm_plan *plan);

/* Replaces pack_a_v2 (im2col/gemm_pack.cpp:192-260) as a one-time step. */
int fc_igemm_pack_filter(fc_context *ctx, const fc_igemm_plan *plan, const float *w_dev,
                         float *Wp_dev, int32_t *table_dev);

/* y[n][k][oh][ow] = sum_{c,r,s} w[k][c][r][s] * x[n][c][oh*sh+r-pt][ow*sw+s-pl].
 * Replaces ConvIm2colLayer::im2col_v1 + sgemm (convLayer/im2colConv.cpp:311-398,
 * 434-565) and the register kernels of im2col/gemm_kernel.cpp; the column matrix
 * is never materialised and y is overwritten (not accumulated).  Layers too small
 * to fill the GPU have plan->split_k > 1: the reduction is cut into parts whose
 * partial sums go to ws_dev (plan->ws_bytes) and are added in a fixed order by a
 * second small kernel; ws_dev may be NULL when plan->ws_bytes is 0. */
int fc_conv_implicit_gemm(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev,
                          const float *Wp_dev, const int32_t *table_dev,
                          const float *bias_dev, int relu, float *ws_dev, float *y_dev);

/* The same layer for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference.  The
 * partial sums of a split reduction go to a static device array of FC_IGEMM_STATIC_WS_BYTES
 * inside the library instead of a workspace of the caller's (each GPU the library runs on holds
 * that array until the process ends); the call allocates nothing and is never bracketed by
 * timing events.  A plan whose ws_bytes exceeds FC_IGEMM_STATIC_WS_BYTES is refused with
 * FC_ERR_UNSUPPORTED.  All calls on one GPU share the array and calls that overlapped in time
 * would race, so one context per GPU uses it at a time: the first context to make this call on a
 * GPU owns the array until fc_destroy, and the call is refused for any other context meanwhile
 * (FC_ERR_STATE); calls of one context are ordered on its stream and safe.  Other processes have
 * their own copy of the array. */
#define FC_IGEMM_STATIC_WS_BYTES (32 << 20)
int fc_conv_implicit_gemm_static(fc_context *ctx, const fc_igemm_plan *plan, const float *x_dev,
                                 const float *Wp_dev, const int32_t *table_dev,
                                 const float *bias_dev, int relu, float *y_dev);

/* ---- recorded launch sequences ----------------------------------------- */

/* Records every launch made on the context between fc_graph_begin and fc_graph_end into a
 * graph that fc_graph_launch replays with one call: for stacks of layers whose kernels are
 * so short that launching them one by one is what takes the time (batch 1).  No counterpart
 * in the reference.  While recording, nothing runs; fc_upload, fc_download, fc_sync and
 * stage timing are refused (FC_ERR_STATE), and the fused and single-kernel Winograd calls
 * must have run once on the context before.  The replay reads and writes the same device
 * buffers as the recorded calls.  fc_graph_destroy waits for the stream first. */
typedef struct fc_graph fc_graph;
int fc_graph_begin(fc_context *ctx);
int fc_graph_end(fc_context *ctx, fc_graph **graph);
int fc_graph_launch(fc_context *ctx, fc_graph *graph);
int fc_graph_destroy(fc_graph *graph);

/* ---- glue for running layers back to back ---------------------------- */

/* 2x2 max pooling, stride 2, NCHW, floor((H)/2) x floor((W)/2) output: the step between
 * the convolution blocks of a VGG-style stack.  No counterpart in the reference (it has
 * no layer but convolution); it exists so that a whole conv trunk can run on the device
 * without host round trips (the layer graph of layer.h:29-84). */
int fc_maxpool2x2(fc_context *ctx, const float *x_dev, float *y_dev, int N, int C, int H, int W);

#ifdef __cplusplus
}
#endif
#endif
