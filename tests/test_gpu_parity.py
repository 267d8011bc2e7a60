"""Parity of the HIP kernels with the CPU oracle, through the C ABI, on a real
MI355X.  Tolerances are the ones the workload definition states:
  * implicit GEMM (im2col path):  max|y-ref| / max|ref| <= 1e-5
  * Winograd F(6,3):              max|y-ref| / max|ref| <= 1e-3
both against the fp64 direct convolution of the oracle on the same seeded
inputs (the fp32 naive result is checked alongside).  Large shapes are covered
by size-independent properties (delta/shift kernels, all-ones closed form,
linearity, agreement of the two algorithms with each other).
"""
import os

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL_IM2COL = 1e-5
TOL_WINO = 1e-3
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "naive_ref_vectors.npz")


@pytest.fixture(scope="module")
def lib():
    import fastconv_amd as F
    L = F.load(0, 20 << 30)
    yield L
    L.close()


def cshape(s):
    import fastconv_amd as F
    return F.ConvShape(*[getattr(s, n) for n, _ in F.ConvShape._fields_])


def announce(*a):
    print(*a, flush=True)


# ------------------------------------------------------------ Winograd stages

@pytest.mark.parametrize("shp,cfg", [
    ((2, 3, 8, 11, 5), 4), ((1, 64, 56, 56, 64), 0), ((3, 10, 14, 14, 70), 3), ((1, 5, 30, 20, 33), 10),
])
def test_winograd_stage_by_stage(lib, shp, cfg):
    s = O.shape(*shp)
    x, w = O.make_inputs(s, seed=1)
    announce("stages", shp, "cfg", cfg)
    y, U, V, M, plan = lib.winograd_conv(cshape(s), x, w, config=cfg, stages=True)
    Uo = O.wino_filter_transform(w)
    Vo = O.wino_input_transform(s, x)
    Mo = O.wino_gemm(Uo, Vo)
    T = plan.T
    # U[f][c][k] against the oracle's U[f][k][c]; padding is exact zeros
    assert np.abs(U[:, :s.C, :s.K].transpose(0, 2, 1) - Uo).max() <= 1e-6 * np.abs(Uo).max()
    assert not U[:, s.C:, :].any() and not U[:, :, s.K:].any()
    assert np.abs(V[:, :s.C, :T] - Vo).max() <= 1e-5 * np.abs(Vo).max()
    assert not V[:, s.C:, :].any() and not V[:, :, T:].any()
    assert np.abs(M[:, :s.K, :T] - Mo).max() <= 1e-5 * np.abs(Mo).max()
    assert not M[:, s.K:, :].any() and not M[:, :, T:].any()
    assert O.max_rel_err(y, O.naive_conv_f64(s, x, w)) <= TOL_WINO


# -------------------------------------------------------- Winograd whole conv

WINO_SHAPES = [
    (1, 64, 56, 56, 64),       # the single-layer case the reference itself runs on a CPU: 64 -> 64 channels at 56x56
    (1, 1, 6, 6, 1), (1, 3, 7, 7, 7), (2, 64, 8, 8, 6), (1, 3, 13, 13, 5), (1, 64, 14, 14, 9),
    (1, 1, 28, 28, 3), (1, 3, 56, 56, 2), (2, 5, 9, 23, 11), (1, 4, 224, 224, 3), (1, 2, 112, 112, 5),
    (5, 7, 7, 7, 130), (32, 16, 14, 14, 16), (3, 130, 28, 28, 40),
]


@pytest.mark.parametrize("shp", WINO_SHAPES)
def test_winograd_against_oracle(lib, shp):
    s = O.shape(*shp)
    x, w = O.make_inputs(s, seed=shp[1] * 7 + shp[2])
    announce("winograd", shp)
    y = lib.winograd_conv(cshape(s), x, w)
    truth = O.naive_conv_f64(s, x, w)
    assert O.max_rel_err(y, truth) <= TOL_WINO
    assert O.max_rel_err(y, O.naive_conv_f32(s, x, w)) <= TOL_WINO
    # and within fp32 rounding of the oracle's own Winograd restatement
    assert O.max_rel_err(y, O.wino_conv_f32(s, x, w)) <= 1e-4


# every 3x3 stride-1 layer of VGG-16 (run_vgg16.sh:5-13) and ResNet-50 (run_resnet50.sh:10-30): (C, K, H)
VGG16_3X3 = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56),
             (256, 512, 28), (512, 512, 28), (512, 512, 14)]
RESNET50_3X3 = [(64, 64, 56), (128, 128, 28), (256, 256, 14), (512, 512, 7)]


@pytest.mark.parametrize("C,K,H", VGG16_3X3 + RESNET50_3X3)
def test_batch1_real_layers_every_path_against_oracle(lib, C, K, H):
    """Batch 1 at the real channel counts: the staged, fused and single-kernel Winograd
    pipelines (<= 1e-3) and the implicit GEMM (<= 1e-5) against the fp64 direct convolution."""
    s = O.shape(1, C, H, H, K)
    cs = cshape(s)
    x, w = O.make_inputs(s, seed=0)
    announce("batch-1 real layer", (C, K, H))
    truth = O.naive_conv_f64(s, x, w)
    assert O.max_rel_err(lib.implicit_gemm_conv(cs, x, w), truth) <= TOL_IM2COL
    assert O.max_rel_err(lib.winograd_conv(cs, x, w), truth) <= TOL_WINO
    assert O.max_rel_err(lib.winograd_conv_fused(cs, x, w), truth) <= TOL_WINO
    if H >= 8:          # a patch row of the single-kernel path is 8 floats of one image row
        assert O.max_rel_err(lib.winograd_conv_onepass(cs, x, w), truth) <= TOL_WINO


RAW_FILTER_SHAPES = [
    (1, 512, 14, 14, 512),      # 9 tiles: the deep VGG-16 layers at batch 1
    (1, 256, 28, 28, 512),      # 25 tiles: two blocks of 16
    (1, 256, 42, 42, 64),       # 49 tiles: four blocks of 16
    (1, 16, 6, 6, 5),           # one tile, one chunk of channels, 5 of 16 output channels
    (2, 48, 12, 12, 20),        # three chunks: the loop tail; output channels not a multiple of 16
    (1, 80, 7, 7, 33),          # five chunks: one pass of the four-deep pipeline plus a tail
    (1, 64, 14, 14, 48),
]


@pytest.mark.parametrize("shp", RAW_FILTER_SHAPES)
def test_winograd_gemm_from_the_untransformed_filter(lib, shp):
    """fc_wino_gemm_raw_filter (U formed in registers from the 3x3 taps) against the oracle's M and,
    through the output transform, the fp64 direct convolution, for every choice of frequencies per
    wavefront and channel split the layer admits."""
    s = O.shape(*shp)
    cs = cshape(s)
    x, w = O.make_inputs(s, seed=shp[1] + shp[4])
    plan = lib.wino_plan(cs, lib.wino_default_config(cs))
    assert lib.wino_raw_filter_gemm_applies(plan)
    T, K, C = plan.T, s.K, s.C
    Mo = O.wino_gemm(O.wino_filter_transform(w), O.wino_input_transform(s, x))
    truth = O.naive_conv_f64(s, x, w)
    nt = 1 if T <= 16 else 2 if T <= 32 else 4
    splits = [sp for sp in (1, 2, 4) if sp <= {1: 4, 2: 2, 4: 1}[nt] and (C // 16) % sp == 0]
    mark = lib.mark()
    try:
        dx, dw = lib.upload(x), lib.upload(w)
        V, M = lib.alloc(plan.V_bytes), lib.alloc(plan.M_bytes)
        y = lib.alloc(4 * s.N * K * plan.OH * plan.OW)
        lib.wino_input_transform(plan, dx, V)
        for fpw, sp in [(0, 0)] + [(f, sp) for f in (1, 2, 4) for sp in splits]:
            announce("raw-filter gemm", shp, "freqs/wave", fpw, "split", sp)
            lib.wino_gemm_raw_filter(plan, dw, V, M, fpw, sp)
            Mh = lib.download(M, (64, plan.K_pad, plan.T_pad))
            assert np.abs(Mh[:, :K, :T] - Mo).max() <= 1e-5 * np.abs(Mo).max()
            lib.wino_output_transform(plan, M, y)
            assert O.max_rel_err(lib.download(y, (s.N, K, plan.OH, plan.OW)), truth) <= TOL_WINO
    finally:
        lib.release(mark)
    # the whole-layer call takes this path by itself when it expects it to win
    assert O.max_rel_err(lib.winograd_conv(cs, x, w), truth) <= TOL_WINO


def test_winograd_gemm_from_the_untransformed_filter_on_random_shapes(lib):
    """Random small geometries (any padding, output channels and tile counts up to 64, channels a multiple of 16)
    through input transform, fc_wino_gemm_raw_filter and output transform against the fp64 direct convolution."""
    rng = np.random.default_rng(7)
    done = 0
    while done < 24:
        N, C, K = int(rng.integers(1, 3)), 16 * int(rng.integers(1, 7)), int(rng.integers(1, 71))
        H, W, pad = int(rng.integers(3, 25)), int(rng.integers(3, 25)), int(rng.integers(0, 3))
        if H + 2 * pad < 3 or W + 2 * pad < 3:
            continue
        s = O.shape(N, C, H, W, K, 3, 3, 1, 1, pad)
        cs = cshape(s)
        plan = lib.wino_plan(cs, lib.wino_default_config(cs))
        if not lib.wino_raw_filter_gemm_applies(plan):
            continue
        done += 1
        x, w = O.make_inputs(s, seed=100 + done)
        announce("raw-filter gemm, random shape", (N, C, H, W, K, pad), "tiles", plan.T)
        mark = lib.mark()
        try:
            dx, dw = lib.upload(x), lib.upload(w)
            V, M = lib.alloc(plan.V_bytes), lib.alloc(plan.M_bytes)
            y = lib.alloc(4 * N * K * plan.OH * plan.OW)
            lib.wino_input_transform(plan, dx, V)
            lib.wino_gemm_raw_filter(plan, dw, V, M)
            lib.wino_output_transform(plan, M, y)
            got = lib.download(y, (N, K, plan.OH, plan.OW))
        finally:
            lib.release(mark)
        assert O.max_rel_err(got, O.naive_conv_f64(s, x, w)) <= TOL_WINO


def test_winograd_gemm_from_the_untransformed_filter_refuses_other_layers(lib):
    import fastconv_amd as F
    for shp in [(1, 24, 14, 14, 32), (4, 64, 56, 56, 64)]:       # channels not a multiple of 16; 400 tiles
        cs = cshape(O.shape(*shp))
        plan = lib.wino_plan(cs, lib.wino_default_config(cs))
        assert not lib.wino_raw_filter_gemm_applies(plan) and not lib.wino_prefer_raw_filter_gemm(plan)
        buf = lib.alloc(1 << 20)
        with pytest.raises(F.FastConvError) as e:
            lib.wino_gemm_raw_filter(plan, buf, buf, buf)
        assert e.value.status == -6
    cs = cshape(O.shape(1, 512, 14, 14, 512))
    plan = lib.wino_plan(cs, lib.wino_default_config(cs))
    assert lib.wino_prefer_raw_filter_gemm(plan)
    buf = lib.alloc(plan.M_bytes)
    for fpw, sp in [(3, 0), (0, 3), (0, 8)]:
        with pytest.raises(F.FastConvError):
            lib.wino_gemm_raw_filter(plan, buf, buf, buf, fpw, sp)


def test_winograd_wide_images(lib):
    """Outputs up to 1020 columns (170 tiles per band) are inside the stated limit of the staged
    pipeline; 512 and 1020 columns take the narrower blocks of the input transform."""
    import fastconv_amd as F
    for (N, C, H, W, K) in [(1, 3, 20, 512, 4), (1, 2, 9, 1020, 3), (2, 5, 14, 640, 6), (1, 4, 7, 760, 2)]:
        s = O.shape(N, C, H, W, K)
        x, w = O.make_inputs(s, seed=W)
        truth = O.naive_conv_f64(s, x, w)
        for cfg in (0, 3, 4):
            announce("wide image", (N, C, H, W, K), "cfg", cfg)
            assert O.max_rel_err(lib.winograd_conv(cshape(s), x, w, config=cfg), truth) <= TOL_WINO
        assert O.max_rel_err(lib.winograd_conv_fused(cshape(s), x, w), truth) <= TOL_WINO
        assert O.max_rel_err(lib.winograd_conv_onepass(cshape(s), x, w), truth) <= TOL_WINO
        assert lib.prefer_winograd(cshape(O.shape(16, 64, H, W, 64)))
    with pytest.raises(F.FastConvError) as e:
        lib.wino_plan(cshape(O.shape(1, 2, 9, 1021, 3)), 0)
    assert e.value.status == -6
    assert not lib.prefer_winograd(cshape(O.shape(16, 64, 9, 1021, 64)))     # auto falls back to implicit GEMM


def test_winograd_every_tile_config(lib):
    s = O.shape(2, 40, 28, 28, 72)
    x, w = O.make_inputs(s, seed=5)
    truth = O.naive_conv_f64(s, x, w)
    for cfg in lib.wino_configs():
        announce("winograd tile config", cfg.id, cfg.bm, cfg.bn, cfg.bk)
        y = lib.winograd_conv(cshape(s), x, w, config=cfg.id)
        assert O.max_rel_err(y, truth) <= TOL_WINO, cfg.id


@pytest.mark.parametrize("pad", [0, 2])
def test_winograd_other_paddings(lib, pad):
    s = O.shape(2, 6, 20, 17, 10, pt=pad)
    x, w = O.make_inputs(s, seed=pad)
    y = lib.winograd_conv(cshape(s), x, w)
    assert y.shape == (2, 10) + O.out_hw(s)
    assert O.max_rel_err(y, O.naive_conv_f64(s, x, w)) <= TOL_WINO


def test_winograd_bias_relu_epilogue(lib):
    s = O.shape(2, 8, 14, 14, 12)
    x, w = O.make_inputs(s, seed=8)
    bias = O.rng_uniform(3, (s.K,))
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    y = lib.winograd_conv(cshape(s), x, w, bias=bias, relu=True)
    assert (y >= 0).all()
    assert O.max_rel_err(y, truth) <= TOL_WINO


def test_nan_and_inf_reach_the_output_of_every_path(lib):
    """A NaN in the input must come out as NaN (not as -inf or 0) wherever it contributes, with ReLU
    off and on (numpy's maximum, which the other tests compare the fused ReLU with, propagates it),
    through the staged, fused, single-kernel and small-channel Winograd epilogues and the implicit
    GEMM (LDS-tiled, with a split reduction, and split over the wavefronts); outputs it does not
    reach stay finite in the implicit GEMM."""
    for shp in [(1, 8, 14, 14, 12), (1, 3, 20, 20, 9)]:
        s = O.shape(*shp)
        cs = cshape(s)
        x, w = O.make_inputs(s, seed=3)
        x[0, 1, 5, 6] = np.nan
        bias = O.rng_uniform(2, (s.K,))
        announce("NaN propagation", shp)
        ws = [c.id for c in lib.igemm_configs() if c.waves_k > 1][0]
        for name, fn in (("staged", lib.winograd_conv), ("fused", lib.winograd_conv_fused),
                         ("single kernel", lib.winograd_conv_onepass), ("implicit gemm", lib.implicit_gemm_conv),
                         ("implicit gemm, LDS-tiled", lambda *a, **k: lib.implicit_gemm_conv(*a, config=3, **k)),
                         ("implicit gemm, wavefront split", lambda *a, **k: lib.implicit_gemm_conv(*a, config=ws, **k))):
            for relu in (False, True):
                y = fn(cs, x, w, bias=bias, relu=relu)
                assert np.isnan(y[0, :, 4:7, 5:8]).all(), (name, relu)          # the 3x3 windows that hold the NaN
                assert not np.isinf(y).any(), (name, relu)
                if name.startswith("implicit gemm"):
                    ok = np.ones(y.shape, bool)
                    ok[0, :, 4:7, 5:8] = False
                    assert np.isfinite(y[ok]).all()


@pytest.mark.parametrize("shp", [
    (2, 3, 8, 11, 5), (1, 64, 56, 56, 64), (3, 10, 14, 14, 70), (2, 16, 7, 7, 33), (1, 8, 30, 20, 40),
    (1, 3, 224, 224, 64), (4, 64, 28, 28, 128), (2, 130, 13, 13, 40),
])
def test_winograd_fused_gemm_output_against_oracle(lib, shp):
    """GEMM + output transform in one kernel (no M buffer): same tolerance as the staged
    pipeline, and the same bits as the staged pipeline (same summation order)."""
    s = O.shape(*shp)
    x, w = O.make_inputs(s, seed=shp[1] + 17)
    bias = O.rng_uniform(3, (s.K,))
    announce("fused winograd", shp)
    y = lib.winograd_conv_fused(cshape(s), x, w, bias=bias, relu=True)
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    assert O.max_rel_err(y, truth) <= TOL_WINO
    assert np.array_equal(y, lib.winograd_conv(cshape(s), x, w, bias=bias, relu=True))


def test_winograd_fused_full_size_layers(lib):
    for (N, C, H, K) in [(32, 3, 224, 64), (32, 64, 112, 128)]:
        s = O.shape(N, C, H, H, K)
        x, w = O.make_inputs(s, seed=2)
        announce("fused full size", (N, C, H, K))
        yf = lib.winograd_conv_fused(cshape(s), x, w)
        yi = lib.implicit_gemm_conv(cshape(s), x, w)
        assert O.max_rel_err(yf, yi) <= TOL_WINO
        sub = O.shape(1, C, H, H, K)
        assert O.max_rel_err(yf[:1], O.naive_conv_f64(sub, np.ascontiguousarray(x[:1]), w)) <= TOL_WINO


@pytest.mark.parametrize("shp,pads", [
    ((2, 3, 8, 11, 5), {}), ((1, 64, 56, 56, 64), {}), ((3, 10, 14, 14, 70), {}), ((2, 16, 7, 8, 33), {}),
    ((1, 8, 30, 20, 40), {}), ((1, 3, 224, 224, 64), {}), ((4, 64, 28, 28, 128), {}), ((2, 21, 13, 13, 40), {}),
    ((2, 6, 20, 17, 10), {"pt": 0}), ((2, 6, 20, 17, 10), {"pt": 2}), ((1, 5, 19, 23, 7), {"pt": 0, "pb": 2, "pl": 2, "pr": 0}),
    ((5, 4, 6, 9, 4), {}), ((1, 1, 3, 8, 1), {}), ((2, 12, 50, 200, 36), {}), ((1, 2, 9, 8, 3), {"pt": 2}),
])
def test_winograd_single_kernel_against_oracle(lib, shp, pads):
    """Input transform, products and output transform in one kernel (neither V nor M exists)."""
    s = O.shape(*shp, **pads)
    x, w = O.make_inputs(s, seed=shp[1] + 29)
    bias = O.rng_uniform(5, (s.K,))
    announce("single-kernel winograd", shp, pads)
    y = lib.winograd_conv_onepass(cshape(s), x, w, bias=bias, relu=True)
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    assert y.shape == truth.shape
    assert O.max_rel_err(y, truth) <= TOL_WINO
    y2 = lib.winograd_conv_onepass(cshape(s), x, w)
    assert O.max_rel_err(y2, O.naive_conv_f64(s, x, w)) <= TOL_WINO


@pytest.mark.parametrize("shp,pads", [
    ((1, 1, 20, 20, 1), {}), ((2, 2, 31, 40, 17), {}), ((3, 3, 45, 45, 64), {}), ((2, 3, 44, 46, 70), {}),
    ((1, 4, 64, 64, 130), {}), ((2, 4, 23, 24, 9), {"pt": 0, "pb": 2, "pl": 2, "pr": 0}), ((7, 3, 32, 32, 32), {}),
    ((1, 3, 100, 372, 5), {}), ((8, 3, 384, 384, 6), {}), ((2, 3, 8, 8, 3), {"pt": 2, "pl": 0}),
])
def test_winograd_small_channel_kernel(lib, shp, pads):
    """Layers with at most four input channels run through a kernel of their own behind the
    single-kernel entry points: every channel count, even and odd output widths (rows stored
    through LDS or every lane its own block), output channels that do not fill a wavefront's
    share, tile counts off the 62 / 64 tiles of a workgroup, 16 and 64 channels per workgroup."""
    s = O.shape(*shp, **pads)
    assert lib.wino_prefer_onepass(cshape(s))
    x, w = O.make_inputs(s, seed=shp[1] + 71)
    bias = O.rng_uniform(9, (s.K,))
    announce("small-channel winograd", shp, pads)
    y = lib.winograd_conv_onepass(cshape(s), x, w, bias=bias, relu=True)
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    assert y.shape == truth.shape
    assert O.max_rel_err(y, truth) <= TOL_WINO
    y2 = lib.winograd_conv_onepass(cshape(s), x, w)
    assert O.max_rel_err(y2, O.naive_conv_f64(s, x, w)) <= TOL_WINO


@pytest.mark.parametrize("shp", [(1, 3, 224, 224, 64), (1, 1, 20, 20, 1), (2, 2, 31, 40, 17), (1, 4, 64, 64, 130),
                                 (2, 3, 44, 46, 70), (1, 3, 30, 30, 9), (32, 3, 64, 64, 64)])
def test_winograd_small_channel_kernel_transforms_the_filter_itself(lib, shp):
    """With few tiles fc_wino_forward_onepass leaves the filter transform to the convolution kernel (one
    launch): the output and the U it leaves behind are those of fc_wino_onepass_filter_transform followed by
    fc_wino_conv_onepass (to rounding), rows and channels of the padding included; a second call with
    filter_ready reads that U and gives the same bits.  (The last shape has enough tiles for the two-launch path.)"""
    s = O.shape(*shp)
    cs = cshape(s)
    x, w = O.make_inputs(s, seed=shp[4] + 5)
    bias = O.rng_uniform(4, (s.K,))
    announce("small-channel winograd, filter transformed in the kernel", shp)
    plan = lib.wino_onepass_plan(cs)
    nU = plan.U_bytes // 4
    mark = lib.mark()
    try:
        dx, dw, db = lib.upload(x), lib.upload(w), lib.upload(bias)
        poison = np.full(nU, 7.0, np.float32)
        U1, U2 = lib.upload(poison), lib.upload(poison)
        y = lib.alloc(4 * s.N * s.K * plan.OH * plan.OW)
        lib.wino_onepass_filter_transform(plan, dw, U1)
        lib.wino_conv_onepass(plan, dx, U1, y, db, True)
        y1 = lib.download(y, (s.N, s.K, plan.OH, plan.OW))
        lib.fill_zero(y, 4 * s.N * s.K * plan.OH * plan.OW)
        lib.wino_forward_onepass(plan, dx, dw, U2, y, db, True)
        y2 = lib.download(y, (s.N, s.K, plan.OH, plan.OW))
        # the same formulas, but the compiler fuses multiplications and additions differently in the two kernels
        assert O.max_rel_err(y2, y1) <= 1e-5
        Ua, Ub = lib.download(U1, (nU,)), lib.download(U2, (nU,))
        assert np.abs(Ua - Ub).max() <= 1e-6 * np.abs(Ua).max()
        assert np.array_equal(Ua == 0.0, Ub == 0.0)          # the zeros of the padding, and nothing left of the 7s
        lib.fill_zero(y, 4 * s.N * s.K * plan.OH * plan.OW)
        lib.wino_forward_onepass(plan, dx, dw, U2, y, db, True, filter_ready=True)
        assert np.array_equal(lib.download(y, (s.N, s.K, plan.OH, plan.OW)), y2)
    finally:
        lib.release(mark)
    assert O.max_rel_err(y1, np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)) <= TOL_WINO


def test_winograd_single_kernel_full_size_layers(lib):
    for (N, C, H, K) in [(32, 3, 224, 64), (32, 64, 112, 128), (8, 64, 224, 64), (32, 64, 224, 64)]:
        s = O.shape(N, C, H, H, K)
        x, w = O.make_inputs(s, seed=2)
        announce("single-kernel full size", (N, C, H, K))
        yf = lib.winograd_conv_onepass(cshape(s), x, w)
        yi = lib.implicit_gemm_conv(cshape(s), x, w)
        assert O.max_rel_err(yf, yi) <= TOL_WINO
        sub = O.shape(1, C, H, H, K)
        assert O.max_rel_err(yf[-1:], O.naive_conv_f64(sub, np.ascontiguousarray(x[-1:]), w)) <= TOL_WINO


def test_pipelines_agree_on_random_shapes(lib):
    """Differential check on 40 seeded random layers: implicit GEMM (the tighter path) against the
    fp64 oracle, and the three Winograd pipelines against it."""
    rng = np.random.default_rng(1234)
    for case in range(40):
        N, C, K = int(rng.integers(1, 4)), int(rng.integers(1, 41)), int(rng.integers(1, 81))
        H, W = int(rng.integers(3, 41)), int(rng.integers(8, 41))
        pt, pb, pl, pr = (int(v) for v in rng.integers(0, 3, size=4))
        if H + pt + pb < 3:
            continue
        s = O.Shape(N, C, H, W, K, 3, 3, 1, 1, pt, pb, pl, pr)
        cs = cshape(s)
        x, w = O.make_inputs(s, seed=case)
        bias = O.rng_uniform(case, (K,))
        announce("random layer", case, (N, C, H, W, K), (pt, pb, pl, pr))
        truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
        yi = lib.implicit_gemm_conv(cs, x, w, bias=bias, relu=True)
        assert O.max_rel_err(yi, truth) <= TOL_IM2COL
        for name, y in (("staged", lib.winograd_conv(cs, x, w, bias=bias, relu=True)),
                        ("fused", lib.winograd_conv_fused(cs, x, w, bias=bias, relu=True)),
                        ("single kernel", lib.winograd_conv_onepass(cs, x, w, bias=bias, relu=True))):
            assert y.shape == truth.shape, name
            assert O.max_rel_err(y, truth) <= TOL_WINO, name


def test_implicit_gemm_on_random_geometries(lib):
    """60 seeded random convolutions (filter 1..5, stride 1..3, asymmetric padding 0..2, channel
    counts around the tile sizes, random tile shape) against the fp64 oracle: whichever of the
    pointwise, unmasked-gather and masked-gather kernels and of the two epilogues a geometry selects."""
    rng = np.random.default_rng(4321)
    ncfg = len(lib.igemm_configs())
    done = 0
    for case in range(80):
        N, C = int(rng.integers(1, 4)), int(rng.choice([1, 3, 8, 16, 20, 32, 48, 64]))
        K = int(rng.choice([1, 7, 32, 64, 72, 128, 256]))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        H, W = int(rng.integers(4, 24)), int(rng.integers(4, 24))
        pt, pb, pl, pr = (int(v) for v in rng.integers(0, 3, size=4))
        if H + pt + pb < kh or W + pl + pr < kw:
            continue
        geo = (N, C, H, W, K, kh, kw, sh, sw, pt, pb, pl, pr)
        s = O.Shape(*geo)
        cfg = int(rng.integers(0, ncfg))
        x, w = O.make_inputs(s, seed=100 + case)
        use_bias, relu = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        bias = O.rng_uniform(case, (K,)) if use_bias else None
        announce("random geometry", case, geo, "tile config", cfg, "bias", use_bias, "relu", relu)
        truth = O.naive_conv_f64(s, x, w, bias)
        if relu:
            truth = np.maximum(truth, 0.0)
        y = lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=relu, config=cfg)
        assert y.shape == truth.shape
        assert O.max_rel_err(y, truth) <= TOL_IM2COL, (case, geo, cfg)
        done += 1
    assert done >= 60


def test_winograd_single_kernel_refuses_narrow_images(lib):
    import fastconv_amd as F
    with pytest.raises(F.FastConvError) as e:
        lib.wino_onepass_plan(cshape(O.shape(1, 4, 12, 7, 4)))
    assert e.value.status == -6
    assert not lib.wino_prefer_onepass(cshape(O.shape(1, 4, 12, 7, 4)))


def test_winograd_single_kernel_plan_is_not_accepted_by_the_staged_calls(lib):
    import fastconv_amd as F
    s = cshape(O.shape(1, 8, 12, 12, 8))
    plan = lib.wino_onepass_plan(s)
    assert plan.V_bytes == 0 and plan.M_bytes == 0 and plan.gemm_config == -1
    buf = lib.alloc(1 << 20)
    with pytest.raises(F.FastConvError):
        lib.wino_filter_transform(plan, buf, buf)
    with pytest.raises(F.FastConvError):
        lib.wino_conv_onepass(lib.wino_plan(s, 0), buf, buf, buf)


def test_winograd_rejects_unsupported(lib):
    import fastconv_amd as F
    for bad in [O.shape(1, 4, 8, 8, 4, 3, 3, 2, 2, 1), O.shape(1, 4, 8, 8, 4, 5, 5, 1, 1, 2),
                O.shape(1, 4, 8, 8, 4, 1, 1, 1, 1, 0)]:
        with pytest.raises(F.FastConvError):
            lib.wino_plan(cshape(bad), 0)


# -------------------------------------------------------------- implicit GEMM

IGEMM_SHAPES = [
    (1, 256, 56, 56, 256, 3, 3, 1, 1, 1),        # the three im2col workload layers: A (3x3, 256 channels at 56x56)
    (1, 128, 56, 56, 256, 3, 3, 2, 2, 1),        # layer B
    (1, 256, 14, 14, 1024, 1, 1, 1, 1, 0),       # layer C
    (1, 3, 224, 224, 64, 7, 7, 2, 2, 3),         # ResNet-50 stem
    (1, 256, 56, 56, 128, 1, 1, 2, 2, 0),        # 1x1 stride-2 projection
    (2, 2048, 7, 7, 512, 1, 1, 1, 1, 0),
    (1, 1, 5, 5, 1, 3, 3, 1, 1, 1), (3, 5, 9, 8, 70, 3, 2, 2, 1, 1), (2, 7, 15, 15, 33, 5, 5, 3, 3, 2),
    # pointwise layers: vector path (pixels per image a multiple of 4) and gather path (7x7 = 49 pixels)
    (32, 64, 56, 56, 256, 1, 1, 1, 1, 0), (3, 70, 6, 6, 33, 1, 1, 1, 1, 0), (5, 20, 7, 7, 40, 1, 1, 1, 1, 0),
    (2, 19, 10, 10, 130, 1, 1, 1, 1, 0),
    # windows that never leave the image (no padding, whole-stage reduction): the gather without bounds masks
    (3, 32, 15, 15, 64, 1, 1, 2, 2, 0), (2, 16, 12, 13, 40, 3, 3, 1, 1, 0), (2, 48, 9, 9, 70, 1, 1, 1, 1, 0),
    (3, 4, 17, 16, 33, 2, 2, 2, 2, 0), (32, 256, 56, 56, 512, 1, 1, 2, 2, 0),
    # ResNet-50 bottleneck layers at batch 32: 1x1 reduce / expand, 3x3 stride 2 (first layer of a stage), the stem
    (32, 256, 56, 56, 64, 1, 1, 1, 1, 0), (32, 512, 28, 28, 128, 1, 1, 1, 1, 0), (32, 2048, 7, 7, 512, 1, 1, 1, 1, 0),
    (32, 1024, 14, 14, 256, 1, 1, 1, 1, 0), (32, 128, 56, 56, 128, 3, 3, 2, 2, 1), (32, 256, 28, 28, 256, 3, 3, 2, 2, 1),
    (32, 512, 14, 14, 512, 3, 3, 2, 2, 1), (8, 3, 224, 224, 64, 7, 7, 2, 2, 3), (32, 3, 224, 224, 64, 7, 7, 2, 2, 3),
    # the 1x1 stride-2 projections (run_resnet50.sh:24,29) at batch 32 and 1; a 3x3 stride-2 layer at batch 1
    (32, 512, 28, 28, 1024, 1, 1, 2, 2, 0), (32, 1024, 14, 14, 2048, 1, 1, 2, 2, 0),
    (1, 512, 28, 28, 1024, 1, 1, 2, 2, 0), (1, 1024, 14, 14, 2048, 1, 1, 2, 2, 0), (1, 256, 28, 28, 256, 3, 3, 2, 2, 1),
    (1, 128, 56, 56, 128, 3, 3, 2, 2, 1), (1, 512, 14, 14, 512, 3, 3, 2, 2, 1),
    # windows of 63, 64 (one 64-bit tap mask) and 81 taps (beyond it: the pointer gather)
    (2, 3, 20, 21, 8, 7, 9, 1, 1, 3), (1, 4, 19, 19, 9, 8, 8, 2, 2, 4), (2, 3, 20, 20, 8, 9, 9, 1, 1, 4),
    # 81 taps with a channel count that is a whole number of stages: the pointer gather over a tap-major filter
    (1, 16, 20, 20, 8, 9, 9, 1, 1, 4), (2, 32, 12, 14, 70, 9, 9, 2, 1, 3),
]


@pytest.mark.parametrize("shp", IGEMM_SHAPES)
def test_implicit_gemm_against_oracle(lib, shp):
    s = O.shape(*shp)
    x, w = O.make_inputs(s, seed=shp[1] + shp[4])
    announce("implicit gemm", shp)
    y = lib.implicit_gemm_conv(cshape(s), x, w)
    assert O.max_rel_err(y, O.naive_conv_f64(s, x, w)) <= TOL_IM2COL
    assert O.max_rel_err(y, O.naive_conv_f32(s, x, w)) <= TOL_IM2COL


def test_implicit_gemm_input_of_2_gib_takes_the_pointer_gather(lib):
    """Inputs below 2 GiB are gathered through a buffer resource with 32-bit offsets; a larger one
    falls back to 64-bit pointers.  One tap per filter gives an exact answer at this size."""
    import fastconv_amd as F
    N, C, H, W, K = 1, 16, 5800, 5800, 2          # 16 channels: a whole stage, so the filter is laid out tap-major
    assert 4 * N * C * H * W >= 1 << 31
    s = O.shape(N, C, H, W, K)
    x = O.rng_uniform(5, (N, C, H, W))
    w = np.zeros((K, C, 3, 3), np.float32)
    w[0, 3, 0, 2] = 1.0
    w[1, 7, 2, 1] = 1.0
    big = F.load(0, 5 << 30)
    try:
        y = big.implicit_gemm_conv(cshape(s), x, w)
    finally:
        big.close()
    xp = np.pad(x[0, 3], 1)
    assert np.array_equal(y[0, 0], xp[0:H, 2:2 + W])
    xp = np.pad(x[0, 7], 1)
    assert np.array_equal(y[0, 1], xp[2:2 + H, 1:1 + W])


def test_implicit_gemm_asymmetric_padding_and_bias(lib):
    s = O.Shape(2, 4, 11, 12, 9, 5, 3, 1, 2, 0, 1, 2, 1)
    x, w = O.make_inputs(s, seed=2)
    bias = O.rng_uniform(4, (s.K,))
    y = lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=True)
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    assert O.max_rel_err(y, truth) <= TOL_IM2COL


def test_implicit_gemm_every_tile_config(lib):
    s = O.shape(2, 24, 19, 19, 72, 3, 3, 2, 2, 1)
    x, w = O.make_inputs(s, seed=6)
    truth = O.naive_conv_f64(s, x, w)
    for cfg in lib.igemm_configs():
        announce("implicit gemm tile config", cfg.id, cfg.bm, cfg.bn, cfg.bk)
        y = lib.implicit_gemm_conv(cshape(s), x, w, config=cfg.id)
        assert O.max_rel_err(y, truth) <= TOL_IM2COL, cfg.id


# every conv geometry of ResNet-50 (run_resnet50.sh:10-30 plus the 3x3 stride-2 variant): (C, K, H, kernel, stride, pad)
RESNET50_GEOMETRIES = [
    (3, 64, 224, 7, 2, 3), (64, 64, 56, 1, 1, 0), (64, 64, 56, 3, 1, 1), (64, 256, 56, 1, 1, 0), (256, 64, 56, 1, 1, 0),
    (256, 128, 56, 1, 1, 0), (128, 128, 56, 3, 2, 1), (128, 128, 28, 3, 1, 1), (128, 512, 28, 1, 1, 0), (512, 128, 28, 1, 1, 0),
    (256, 512, 56, 1, 2, 0), (512, 256, 28, 1, 1, 0), (256, 256, 28, 3, 2, 1), (256, 256, 14, 3, 1, 1), (256, 1024, 14, 1, 1, 0),
    (1024, 256, 14, 1, 1, 0), (512, 1024, 28, 1, 2, 0), (1024, 512, 14, 1, 1, 0), (512, 512, 14, 3, 2, 1), (512, 512, 7, 3, 1, 1),
    (512, 2048, 7, 1, 1, 0), (2048, 512, 7, 1, 1, 0), (1024, 2048, 14, 1, 2, 0),
]


@pytest.mark.parametrize("geo", RESNET50_GEOMETRIES)
def test_implicit_gemm_batch1_resnet50_layers(lib, geo):
    """Batch 1, the library's untuned choice: against the fp64 oracle at 1e-5, the same bits on a second run,
    and (but for the layers that fill the chip unsplit) one launch with the reduction split inside the workgroups."""
    C, K, H, ks, st, pad = geo
    s = O.shape(1, C, H, H, K, ks, ks, st, st, pad)
    cs = cshape(s)
    cfg = lib.igemm_default_config(cs)
    g = lib.igemm_configs()[cfg]
    plan = lib.igemm_plan(cs, cfg)
    announce("batch-1 ResNet-50 layer", geo, "tile %dx%d, %d wavefronts over the reduction, split %d" % (g.bm, g.bn, g.waves_k, plan.split_k))
    if C % 16 == 0 and (C, K, H, ks) not in ((64, 64, 56, 1), (64, 256, 56, 1)):
        assert g.waves_k > 1 and plan.split_k == 1 and plan.ws_bytes == 0
    x, w = O.make_inputs(s, seed=C + K)
    bias = O.rng_uniform(K, (K,))
    y1 = lib.implicit_gemm_conv(cs, x, w, bias=bias, relu=True)
    y2 = lib.implicit_gemm_conv(cs, x, w, bias=bias, relu=True)
    assert np.array_equal(y1, y2)
    assert O.max_rel_err(y1, np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)) <= TOL_IM2COL
    assert O.max_rel_err(lib.implicit_gemm_conv(cs, x, w), O.naive_conv_f64(s, x, w)) <= TOL_IM2COL


WAVESPLIT_SHAPES = [
    # tap-major, windows inside the image (1x1, unpadded 3x3, stride 2): pixel blocks that end inside an image and span two
    (1, 32, 7, 7, 40, 1, 1, 1, 1, 0), (3, 16, 9, 10, 33, 1, 1, 2, 2, 0), (2, 48, 11, 9, 20, 3, 3, 1, 1, 0), (1, 64, 13, 13, 64, 2, 2, 2, 2, 0),
    # tap-major with padding (taps outside the image are refused by the buffer's range check)
    (1, 16, 7, 7, 16, 3, 3, 1, 1, 1), (2, 32, 14, 14, 48, 3, 3, 2, 2, 1), (1, 80, 5, 6, 17, 5, 5, 1, 1, 2), (1, 16, 12, 12, 8, 7, 7, 2, 2, 3),
    # channel counts that are not whole units: the row table
    (2, 24, 9, 9, 30, 3, 3, 1, 1, 1), (1, 3, 20, 20, 10, 7, 7, 2, 2, 3), (3, 5, 8, 8, 70, 1, 1, 1, 1, 0), (1, 1, 6, 6, 1, 3, 3, 1, 1, 1),
    # fewer reduction units than wavefronts; one pixel
    (1, 16, 4, 4, 16, 1, 1, 1, 1, 0), (1, 32, 1, 1, 9, 1, 1, 1, 1, 0), (1, 16, 3, 3, 5, 3, 3, 1, 1, 0),
]


@pytest.mark.parametrize("shp", WAVESPLIT_SHAPES)
def test_implicit_gemm_reduction_split_inside_the_workgroup(lib, shp):
    """Every configuration of the kernels that split the reduction over the wavefronts of a workgroup, with
    bias and ReLU, against the fp64 oracle."""
    s = O.shape(*shp)
    x, w = O.make_inputs(s, seed=shp[1] + 3 * shp[4])
    bias = O.rng_uniform(6, (s.K,))
    truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
    n = 0
    for cfg in lib.igemm_configs():
        if cfg.waves_k == 1:
            continue
        announce("wavefront-split reduction", shp, "tile %dx%d, %d wavefronts" % (cfg.bm, cfg.bn, cfg.waves_k))
        plan = lib.igemm_plan(cshape(s), cfg.id)
        assert plan.split_k == 1 and plan.ws_bytes == 0
        y = lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=True, config=cfg.id)
        assert y.shape == truth.shape
        assert O.max_rel_err(y, truth) <= TOL_IM2COL, cfg.id
        n += 1
    assert n >= 12


def test_implicit_gemm_wavefront_split_refuses_what_it_cannot_address(lib):
    """These kernels address x with one 32-bit offset (bit 31 spare) and one 64-bit mask of taps: larger layers
    are refused at plan time and the untuned choice stays with the LDS-tiled kernels."""
    import fastconv_amd as F
    ws = [c.id for c in lib.igemm_configs() if c.waves_k > 1]
    for bad in [O.shape(1, 16, 5800, 5800, 2), O.shape(2, 3, 20, 20, 8, 9, 9, 1, 1, 4)]:
        with pytest.raises(F.FastConvError) as e:
            lib.igemm_plan(cshape(bad), ws[0])
        assert e.value.status == -6
        assert lib.igemm_configs()[lib.igemm_default_config(cshape(bad))].waves_k == 1


def test_implicit_gemm_full_tile_epilogue_paths(lib):
    """Output-channel counts that are whole tiles take the predicate-free epilogue (plain, and
    with bias / ReLU); pixel blocks that straddle images and end inside a block are part of it."""
    for shp in [(3, 32, 13, 13, 256, 1, 1, 1, 1, 0), (2, 48, 17, 17, 256, 3, 3, 2, 2, 1), (5, 64, 14, 14, 256, 1, 1, 1, 1, 0)]:
        s = O.shape(*shp)
        x, w = O.make_inputs(s, seed=8)
        bias = O.rng_uniform(12, (s.K,))
        plain = O.naive_conv_f64(s, x, w)
        with_bias = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
        only_bias = O.naive_conv_f64(s, x, w, bias)
        for cfg in lib.igemm_configs():
            announce("full-tile epilogue", shp, "tile", cfg.bm, cfg.bn)
            assert O.max_rel_err(lib.implicit_gemm_conv(cshape(s), x, w, config=cfg.id), plain) <= TOL_IM2COL
            assert O.max_rel_err(lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=True, config=cfg.id),
                                 with_bias) <= TOL_IM2COL
            assert O.max_rel_err(lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, config=cfg.id),
                                 only_bias) <= TOL_IM2COL


def test_implicit_gemm_split_reduction_is_exact_and_repeatable(lib):
    """Under the LDS-tiled 64x64 shape batch-1 layers are too few workgroups to fill the GPU: their
    reduction is split over workgroups and the parts are added in a fixed order by a second kernel, so
    two runs give the same bits."""
    for shp in [(1, 2048, 7, 7, 512, 1, 1, 1, 1, 0), (1, 256, 56, 56, 256, 3, 3, 1, 1, 1),
                (1, 512, 14, 14, 512, 3, 3, 2, 2, 1), (1, 1024, 14, 14, 256, 1, 1, 1, 1, 0)]:
        s = O.shape(*shp)
        plan = lib.igemm_plan(cshape(s), 3)
        assert plan.split_k > 1, shp
        x, w = O.make_inputs(s, seed=3)
        bias = O.rng_uniform(9, (s.K,))
        announce("split reduction", shp, "parts", plan.split_k)
        y1 = lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=True, config=3)
        y2 = lib.implicit_gemm_conv(cshape(s), x, w, bias=bias, relu=True, config=3)
        assert np.array_equal(y1, y2)
        truth = np.maximum(O.naive_conv_f64(s, x, w, bias), 0.0)
        assert O.max_rel_err(y1, truth) <= TOL_IM2COL


# ------------------------------------------- the reference's own naive layers

def test_golden_vectors_of_reference_naive_layers(lib):
    z = np.load(GOLD)
    names = sorted({k.split("/")[0] for k in z.files})
    for name in names:
        if name + "/bias_elems" in z.files:
            continue                 # per-element bias tensor: not a fast-path feature
        s = O.Shape(*[int(v) for v in z[name + "/shape"]])
        x, w, y_ref = z[name + "/x"], z[name + "/w"], z[name + "/y"]
        announce("golden", name)
        y = lib.implicit_gemm_conv(cshape(s), x, w)
        assert O.max_rel_err(y, y_ref) <= TOL_IM2COL, name
        if s.kh == 3 and s.kw == 3 and s.sh == 1 and s.sw == 1:
            yw = lib.winograd_conv(cshape(s), x, w)
            assert O.max_rel_err(yw, y_ref) <= TOL_WINO, name


# ------------------------------------------------ full-size layers: properties

def _full_layers():
    # (N, C, H, K): VGG-16 and ResNet-50 3x3 stride-1 layers at batch 32
    return [(32, 3, 224, 64), (32, 64, 224, 64), (32, 64, 112, 128), (32, 128, 112, 128), (32, 128, 56, 256),
            (32, 256, 56, 256), (32, 256, 28, 512), (32, 512, 28, 512), (32, 512, 14, 512),
            (32, 64, 56, 64), (32, 128, 28, 128), (32, 256, 14, 256), (32, 512, 7, 512)]


@pytest.mark.parametrize("N,C,H,K", _full_layers())
def test_full_size_shift_kernel_property(lib, N, C, H, K):
    """With w[k][c] = delta(c == k % C) * one tap at (u, v), output channel k is
    input channel k % C shifted by (u-1, v-1): an exact answer at any size."""
    s = O.shape(N, C, H, H, K)
    x = O.rng_uniform(11, (N, C, H, H))
    u, v = 2, 0
    w = np.zeros((K, C, 3, 3), np.float32)
    w[np.arange(K), np.arange(K) % C, u, v] = 1.0
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    expect = xp[:, np.arange(K) % C, u:u + H, v:v + H]
    announce("full-size shift", (N, C, H, K))
    yw = lib.winograd_conv(cshape(s), x, w)
    assert O.max_rel_err(yw, expect) <= TOL_WINO
    yi = lib.implicit_gemm_conv(cshape(s), x, w)
    assert np.array_equal(yi, expect)            # one non-zero product per output: exact


@pytest.mark.parametrize("N,C,H,K", [(32, 256, 56, 256), (32, 64, 224, 64), (32, 512, 14, 512), (32, 128, 56, 256),
                                     (32, 256, 28, 512), (32, 128, 28, 128), (32, 256, 14, 256)])
def test_full_size_two_algorithms_agree_and_are_linear(lib, N, C, H, K):
    s = O.shape(N, C, H, H, K)
    x, w = O.make_inputs(s, seed=1)
    announce("full-size agreement", (N, C, H, K))
    yw = lib.winograd_conv(cshape(s), x, w)
    yi = lib.implicit_gemm_conv(cshape(s), x, w)
    assert O.max_rel_err(yw, yi) <= TOL_WINO
    # spot-check 3 images' worth of output channels against the fp64 oracle
    sub = O.shape(1, C, H, H, K)
    truth = O.naive_conv_f64(sub, np.ascontiguousarray(x[N - 1:N]), w)
    assert O.max_rel_err(yi[N - 1:N], truth) <= TOL_IM2COL
    assert O.max_rel_err(yw[N - 1:N], truth) <= TOL_WINO
    # linearity in the input: conv(2x) == 2 conv(x) exactly in binary floating point
    y2 = lib.winograd_conv(cshape(s), 2.0 * x, w)
    assert np.array_equal(y2, 2.0 * yw)


def test_all_ones_closed_form_full_size(lib):
    s = O.shape(32, 128, 112, 112, 128)
    x = np.ones((s.N, s.C, s.H, s.W), np.float32)
    w = np.ones((s.K, s.C, 3, 3), np.float32)
    cnt = np.full((112, 112), 9.0)
    cnt[0, :] = cnt[-1, :] = cnt[:, 0] = cnt[:, -1] = 6.0
    cnt[0, 0] = cnt[0, -1] = cnt[-1, 0] = cnt[-1, -1] = 4.0
    expect = np.broadcast_to(s.C * cnt, (s.N, s.K, 112, 112))
    yi = lib.implicit_gemm_conv(cshape(s), x, w)
    assert np.array_equal(yi, expect)
    yw = lib.winograd_conv(cshape(s), x, w)
    assert O.max_rel_err(yw, expect) <= TOL_WINO


# ------------------------------------------- large batches (64 and 128 images)

@pytest.mark.parametrize("N", [64, 128])
@pytest.mark.parametrize("C,H", [(256, 56), (512, 28), (512, 14)])
def test_large_batch_stress_layers(lib, N, C, H):
    """The throughput-stress layers at batch 64 and 128, through the staged pipeline (whole-layer
    U, V, M), the blocked one (no M) and the implicit GEMM: an exact shift-kernel answer, agreement
    of the three paths on seeded data, and the first and last image against the fp64 oracle."""
    K = C
    s = O.shape(N, C, H, H, K)
    cs = cshape(s)
    announce("stress layer", (N, C, H, K))
    x = O.rng_uniform(21, (N, C, H, H))
    u, v = 0, 2
    wd = np.zeros((K, C, 3, 3), np.float32)
    wd[np.arange(K), (np.arange(K) * 7 + 3) % C, u, v] = 1.0
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    expect = xp[:, (np.arange(K) * 7 + 3) % C, u:u + H, v:v + H]
    assert np.array_equal(lib.implicit_gemm_conv(cs, x, wd), expect)
    assert O.max_rel_err(lib.winograd_conv(cs, x, wd), expect) <= TOL_WINO
    assert O.max_rel_err(lib.winograd_conv_fused(cs, x, wd), expect) <= TOL_WINO
    del xp, expect
    _, w = O.make_inputs(O.shape(1, C, H, H, K), seed=4)
    yi = lib.implicit_gemm_conv(cs, x, w)
    ys = lib.winograd_conv(cs, x, w)
    assert O.max_rel_err(ys, yi) <= TOL_WINO
    yb = lib.winograd_conv_fused(cs, x, w)
    assert np.array_equal(yb, ys)          # same products in the same order, M kept in registers instead of HBM
    sub = O.shape(1, C, H, H, K)
    for n in (0, N - 1):
        truth = O.naive_conv_f64(sub, np.ascontiguousarray(x[n:n + 1]), w)
        assert O.max_rel_err(yi[n:n + 1], truth) <= TOL_IM2COL
        assert O.max_rel_err(ys[n:n + 1], truth) <= TOL_WINO


# ------------------------------------------------------- recorded sequences

def test_recorded_graph_replays_match_eager_results(lib):
    """Three layers (staged Winograd with the online filter transform, the single-kernel path,
    an implicit GEMM that splits its reduction) recorded once; every replay, with fresh inputs and
    eager work in between, must give the bits of the eager run on the same inputs."""
    import fastconv_amd as F
    s1, s2, s3 = cshape(O.shape(2, 24, 20, 20, 40)), cshape(O.shape(2, 40, 20, 20, 16)), \
        cshape(O.Shape(2, 16, 20, 20, 48, 3, 3, 2, 2, 1, 1, 1, 1))
    p1, p2 = lib.wino_plan(s1, 3), lib.wino_onepass_plan(s2)
    p3 = lib.igemm_plan(s3, 0)
    assert p3.split_k > 1
    w1, w2, w3 = (O.rng_normal(i, shp, 0.1) for i, shp in ((1, (40, 24, 3, 3)), (2, (16, 40, 3, 3)), (3, (48, 16, 3, 3))))
    dw1, dw2, dw3 = lib.upload(w1), lib.upload(w2), lib.upload(w3)
    x = lib.alloc(4 * 2 * 24 * 20 * 20)
    U1, V1, M1 = lib.alloc(p1.U_bytes), lib.alloc(p1.V_bytes), lib.alloc(p1.M_bytes)
    y1 = lib.alloc(4 * 2 * 40 * 20 * 20)
    U2, y2 = lib.alloc(p2.U_bytes), lib.alloc(4 * 2 * 16 * 20 * 20)
    Wp, tab, ws = lib.alloc(p3.Wp_bytes), lib.alloc(p3.table_bytes), lib.alloc(p3.ws_bytes)
    y3 = lib.alloc(4 * 2 * 48 * 10 * 10)
    lib.igemm_pack_filter(p3, dw3, Wp, tab)

    def run():
        lib.wino_forward(p1, x, dw1, U1, V1, M1, y1, relu=True)
        lib.wino_forward_onepass(p2, y1, dw2, U2, y2, relu=True)
        lib.conv_implicit_gemm(p3, y2, Wp, tab, y3, ws=ws)

    def fresh(seed):
        lib.upload_into(x, O.rng_uniform(seed, (2, 24, 20, 20)))

    fresh(10)
    run()                       # also grants the large LDS sizes before recording
    lib.sync()
    lib.graph_begin()
    with pytest.raises(F.FastConvError):
        lib.sync()              # refused while recording
    run()
    g = lib.graph_end()
    try:
        for seed in (11, 12, 13):
            fresh(seed)
            run()
            eager = lib.download(y3, (2, 48, 10, 10))
            lib.fill_zero(y3, 4 * 2 * 48 * 10 * 10)
            lib.fill_zero(M1, p1.M_bytes)
            lib.sync()
            lib.graph_launch(g)
            replay = lib.download(y3, (2, 48, 10, 10))
            assert np.abs(eager).max() > 0
            assert np.array_equal(eager, replay), seed
    finally:
        lib.graph_destroy(g)


# ----------------------------------------------------------------- the arena

def test_pool_exhaustion_is_reported(lib):
    import fastconv_amd as F
    cap, used, _ = lib.pool_stats()
    with pytest.raises(F.FastConvError) as e:
        lib.alloc(cap + 1)
    assert e.value.status == -4
    assert lib.pool_stats()[1] == used


def test_stage_timers_count_launches(lib):
    s = O.shape(1, 8, 12, 12, 8)
    x, w = O.make_inputs(s)
    lib.timing(True)
    lib.timing_reset()
    lib.winograd_conv(cshape(s), x, w)
    lib.winograd_conv(cshape(s), x, w)
    # the whole-layer call puts filter and input transform into one launch, booked as stage 1
    assert lib.stage_time(0)[1] == 0
    for stage in (1, 2, 3):
        ms, cnt = lib.stage_time(stage)
        assert cnt == 2 and ms > 0.0
    plan = lib.wino_plan(cshape(s), 0)
    buf = lib.alloc(max(plan.U_bytes, 4096))
    lib.wino_filter_transform(plan, lib.upload(w), buf)
    assert lib.stage_time(0)[1] == 1
    lib.timing(False)


def test_clock_probe_reports_a_plausible_shader_clock(lib):
    import fastconv_amd as F
    s = O.shape(4, 64, 56, 56, 64)
    x, w = O.make_inputs(s, seed=2)
    ref = lib.winograd_conv(cshape(s), x, w)
    with pytest.raises(F.FastConvError):
        lib.clock_probe_end()                   # nothing running
    with pytest.raises(F.FastConvError):
        lib.clock_probe_begin(0, 100)
    with pytest.raises(F.FastConvError):
        lib.clock_probe_begin(8, 0)
    lib.clock_probe_begin(12, 200)
    with pytest.raises(F.FastConvError):
        lib.clock_probe_begin(4, 100)           # one at a time
    y = lib.winograd_conv(cshape(s), x, w)      # work beside the probe is not disturbed
    mhz = lib.clock_probe_end()
    announce("shader clock samples (MHz):", [round(v) for v in mhz])
    assert len(mhz) == 12 and all(300.0 < v < 3000.0 for v in mhz)
    np.testing.assert_array_equal(y, ref)
    lib.clock_probe_begin(2, 50)                # usable again
    assert len(lib.clock_probe_end()) == 2


def test_filter_and_input_transform_in_one_launch_match_the_two_launches(lib):
    for shp in [(2, 3, 8, 11, 5), (1, 64, 56, 56, 64), (3, 10, 14, 14, 70), (1, 5, 30, 200, 33)]:
        s = cshape(O.shape(*shp))
        x, w = O.make_inputs(O.shape(*shp), seed=5)
        for cfg in (0, 4, 10):
            plan = lib.wino_plan(s, cfg)
            mark = lib.mark()
            dx, dw = lib.upload(x), lib.upload(w)
            U1, V1, U2, V2 = (lib.alloc(plan.U_bytes), lib.alloc(plan.V_bytes), lib.alloc(plan.U_bytes),
                              lib.alloc(plan.V_bytes))
            lib.wino_filter_transform(plan, dw, U1)
            lib.wino_input_transform(plan, dx, V1)
            lib.wino_filter_input_transform(plan, dw, U2, dx, V2)
            ushape, vshape = (64, plan.C_pad, plan.K_pad), (64, plan.C_pad, plan.T_pad)
            assert np.array_equal(lib.download(U1, ushape), lib.download(U2, ushape))
            assert np.array_equal(lib.download(V1, vshape), lib.download(V2, vshape))
            lib.release(mark)


# ------------------------------------------ untuned choices away from the layers they were fitted on

def _launch_us(lib, fn, iters=20, rounds=3):
    import time
    fn()
    lib.sync()
    best = 1e30
    for _ in range(rounds):
        t0 = time.perf_counter()
        for _ in range(iters):
            fn()
        lib.sync()
        best = min(best, (time.perf_counter() - t0) / iters * 1e6)
    return best


@pytest.mark.parametrize("geo", [
    (8, 96, 35, 35, 192, 3, 1, 1), (32, 160, 17, 17, 160, 3, 1, 1), (4, 48, 112, 112, 48, 3, 1, 1),
    (16, 320, 28, 28, 64, 1, 1, 0), (8, 96, 57, 57, 96, 3, 2, 1),
])
def test_untuned_tile_choice_is_close_to_the_best_of_a_search(lib, geo):
    """Shapes that none of the default rules was fitted on: the configuration the library picks without tuning
    (fc_wino_gemm_default_config for the staged Winograd pipeline, fc_igemm_default_config for the implicit GEMM)
    takes at most 10 % (Winograd) or 15 % (implicit GEMM, whose search has 25 configurations and 10-20 us launches;
    measured 0-9 %) longer than the best configuration of a search over all of them (20 launches back to back, best
    of three rounds)."""
    N, C, H, W, K, ks, st, pad = geo
    s = O.shape(N, C, H, W, K, ks, ks, st, st, pad)
    cs = cshape(s)
    x, w = O.make_inputs(s, seed=1)
    mark = lib.mark()
    try:
        dx, dw = lib.upload(x), lib.upload(w)
        oh, ow = O.out_hw(s)
        y = lib.alloc(4 * N * K * oh * ow)
        if ks == 3 and st == 1:
            times = {}
            for g in lib.wino_configs():
                plan = lib.wino_plan(cs, g.id)
                if plan.K_pad > 2 * K and g.bm > 32:
                    continue
                m2 = lib.mark()
                U, V, M = lib.alloc(plan.U_bytes), lib.alloc(plan.V_bytes), lib.alloc(plan.M_bytes)
                times[g.id] = _launch_us(lib, lambda: lib.wino_forward(plan, dx, dw, U, V, M, y))
                lib.release(m2)
            d = lib.wino_default_config(cs)
            announce("winograd", geo, "untuned config", d, "%.1f us" % times[d], "best", min(times, key=times.get), "%.1f us" % min(times.values()))
            assert times[d] <= 1.10 * min(times.values()), (geo, times)
        times = {}
        for g in lib.igemm_configs():
            try:
                plan = lib.igemm_plan(cs, g.id)
            except Exception:
                continue
            m2 = lib.mark()
            Wp, tab = lib.alloc(plan.Wp_bytes), lib.alloc(plan.table_bytes)
            ws = lib.alloc(plan.ws_bytes) if plan.ws_bytes else None
            lib.igemm_pack_filter(plan, dw, Wp, tab)
            times[g.id] = _launch_us(lib, lambda: lib.conv_implicit_gemm(plan, dx, Wp, tab, y, ws=ws))
            lib.release(m2)
        d = lib.igemm_default_config(cs)
        announce("implicit gemm", geo, "untuned config", d, "%.1f us" % times[d], "best", min(times, key=times.get), "%.1f us" % min(times.values()))
        assert times[d] <= 1.15 * min(times.values()), (geo, times)
    finally:
        lib.release(mark)
