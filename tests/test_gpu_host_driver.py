"""The C++ host side on a real MI355X: the ConvTest driver over the three layer classes
(check against the host naive convolution, the reference's own acceptance test), Tuning(),
and the layer graph running a VGG-16 style trunk back to back on the device."""
import os
import re
import subprocess

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "fastconv_amd")


def _exe(name):
    path = os.path.join(PKG, "bin", name)
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", PKG, "-s", "host"])
    return path


def _run(args, cwd=None):
    print(" ".join(args), flush=True)
    r = subprocess.run(args, capture_output=True, text=True, timeout=110, cwd=cwd)
    assert r.returncode == 0, r.stdout + r.stderr
    return r.stdout


@pytest.mark.parametrize("algo", [["-a", "winograd"], ["-a", "winograd", "--variant", "blocked"],
                                  ["-a", "winograd", "-ts", "offline"], ["-a", "im2col"], ["-a", "auto"]])
def test_conv_test_driver_passes_its_own_check(algo):
    out = _run([_exe("conv_test"), "-ic", "16", "-oc", "24", "-is", "28", "28", "-ks", "3", "3", "-ip", "1",
                "-n", "2", "-i", "3", "--strict"] + algo)
    assert "PASS" in out and "FAIL" not in out


@pytest.mark.parametrize("ts", ["online", "offline"])
@pytest.mark.parametrize("C,H", [(512, 14), (256, 28)])
def test_batch1_deep_layers_through_the_staged_layer_class(ts, C, H):
    """Batch 1 with 9 and 25 tiles through ConvWinoF63ZCLayer: with the online filter transform the
    products are made straight from the 3x3 filter, with the offline one from the transformed filter."""
    out = _run([_exe("conv_test"), "-ic", str(C), "-oc", "512", "-is", str(H), str(H), "-ks", "3", "3", "-ip", "1",
                "-n", "1", "-i", "3", "-t", "16", "-a", "winograd", "-ts", ts, "--strict", "--json"])
    assert "PASS" in out and "FAIL" not in out
    j = _json_line(out)
    assert j["max_rel_err"] <= 1e-3 and j["kernel_transform"] == ts


def _json_line(out):
    import json
    return json.loads([l for l in out.splitlines() if l.startswith("{")][-1])


def test_json_line_reports_every_stage_against_its_roofline():
    """conv_test --json: per-stage rates and their fraction of the fp32 MFMA peak (GEMM stages) or of the HBM
    peak (transforms), consistent with the stage times on the same line."""
    base = [_exe("conv_test"), "-ic", "128", "-oc", "128", "-is", "56", "56", "-ks", "3", "3", "-ip", "1", "-n", "8",
            "-i", "5", "-t", "16", "--check-images", "1", "--strict", "--json"]
    j = _json_line(_run(base + ["-a", "winograd", "--variant", "zc"]))
    assert j["peak_mfma_tflops"] == 157.3 and j["peak_hbm_gbs"] == 8000
    T = 8 * 10 * 10
    assert j["gemm_tflops"] == pytest.approx(2 * 64 * 128 * 128 * T / (j["gemm_ms"] * 1e-3) / 1e12, rel=1e-2)
    assert j["gemm_frac_mfma"] == pytest.approx(j["gemm_tflops"] / 157.3, abs=2e-4)
    assert j["input_tran_gbs"] == pytest.approx((4 * 8 * 128 * 56 * 56 + 256 * 128 * T) / (j["input_tran_ms"] * 1e-3) / 1e9, rel=1e-2)
    assert j["output_tran_gbs"] == pytest.approx((256 * 128 * T + 4 * 8 * 128 * 56 * 56) / (j["output_tran_ms"] * 1e-3) / 1e9, rel=1e-2)
    for k in ("gemm_frac_mfma", "input_tran_frac_hbm", "output_tran_frac_hbm"):
        assert 0.0 < j[k] < 1.0, k
    j = _json_line(_run(base + ["-a", "im2col"]))
    assert j["gemm_tflops"] == pytest.approx(2 * 8 * 128 * 128 * 56 * 56 * 9 / (j["gemm_ms"] * 1e-3) / 1e12, rel=1e-2)
    assert 0.0 < j["gemm_frac_mfma"] < 1.0 and j["input_tran_gbs"] is None and j["output_tran_frac_hbm"] is None


@pytest.mark.parametrize("variant", ["zc", "blocked"])
@pytest.mark.parametrize("batch,C,H", [(64, 256, 56), (128, 256, 56), (64, 512, 28), (128, 512, 28), (64, 512, 14),
                                       (128, 512, 14)])
def test_stress_layers_through_both_winograd_layer_classes_with_tuning(tmp_path, variant, batch, C, H):
    """Batch 64 / 128 on the throughput-stress layers through ConvWinoF63ZCLayer (staged, whole-layer
    buffers) and ConvWinoF63Layer (blocked) with -tn tuning; the driver's own check covers the last
    image of the batch (the host convolution of 128 images would take minutes)."""
    out = _run([_exe("conv_test"), "-ic", str(C), "-oc", str(C), "-is", str(H), str(H), "-ks", "3", "3", "-ip", "1",
                "-n", str(batch), "-i", "2", "-t", "16", "-a", "winograd", "--variant", variant, "-tn", "tuning",
                "--check-images", "1", "--strict", "--json"], cwd=str(tmp_path))
    assert "PASS" in out and "FAIL" not in out and "Best Config" in out
    j = _json_line(out)
    assert j["batch"] == batch and j["checked_images"] == 1 and j["max_rel_err"] <= 1e-3
    assert j["algorithm"] == ("winograd_blocked" if variant == "blocked" else "winograd")
    assert j["kernel_transform"] in ("online", "offline")


@pytest.mark.parametrize("geo", [
    # ResNet-50 (run_resnet50.sh:10-30 and the 3x3 stride-2 variant): ic, oc, size, kernel, stride, pad
    (64, 64, 56, 3, 1, 1), (128, 128, 28, 3, 1, 1), (256, 256, 14, 3, 1, 1), (512, 512, 7, 3, 1, 1),
    (256, 64, 56, 1, 1, 0), (64, 256, 56, 1, 1, 0), (512, 128, 28, 1, 1, 0), (1024, 256, 14, 1, 1, 0),
    (2048, 512, 7, 1, 1, 0), (128, 128, 56, 3, 2, 1), (3, 64, 224, 7, 2, 3)])
@pytest.mark.parametrize("batch", [1, 32])
def test_auto_algorithm_on_resnet50_layers(geo, batch):
    ic, oc, size, ks, st, pad = geo
    out = _run([_exe("conv_test"), "-ic", str(ic), "-oc", str(oc), "-is", str(size), str(size), "-ks", str(ks), str(ks),
                "-s", str(st), str(st), "-ip", str(pad), "-n", str(batch), "-i", "2", "-t", "16", "-a", "auto",
                "--check-images", "1", "--strict", "--json"])
    assert "PASS" in out and "FAIL" not in out
    j = _json_line(out)
    # the driver's choice is the library's rule (3x3 stride 1) inside the reference's skeleton
    from fastconv_amd import capi
    import ctypes
    shape = capi.ConvShape(batch, ic, size, size, oc, ks, ks, st, st, pad, pad, pad, pad)
    want = "winograd" if capi.load_cdll().fc_prefer_winograd(ctypes.byref(shape)) else "im2col"
    if ks == 1 and st == 1:
        want = "direct"
    if batch == 32 and ks == 3 and st == 1:
        assert want == "winograd"
    assert j["algorithm"].split("_")[0] == want, j
    assert j["max_rel_err"] <= (1e-3 if want == "winograd" else 1e-5)


def test_blocked_variant_honours_the_transform_strategy():
    base = [_exe("conv_test"), "-ic", "16", "-oc", "24", "-is", "28", "28", "-ks", "3", "3", "-n", "2", "-i", "2",
            "--strict", "--json", "-a", "winograd", "--variant", "blocked"]
    on = _json_line(_run(base))
    off = _json_line(_run(base + ["-ts", "offline"]))
    assert on["kernel_transform"] == "online" and off["kernel_transform"] == "offline"
    assert on["kernel_tran_ms"] > 0.0 and off["kernel_tran_ms"] == 0.0


def test_conv_test_pointwise_and_strided_go_to_implicit_gemm():
    out = _run([_exe("conv_test"), "-ic", "32", "-oc", "16", "-is", "14", "14", "-ks", "1", "1", "-a", "auto",
                "-i", "2", "--strict"])
    assert "PASS" in out
    out = _run([_exe("conv_test"), "-ic", "3", "-oc", "8", "-is", "32", "32", "-ks", "7", "7", "-ip", "3", "-s", "2", "2",
                "-a", "im2col", "-i", "2", "--strict"])
    assert "PASS" in out


def test_tuning_writes_a_log_that_the_next_run_uses(tmp_path):
    exe = _exe("conv_test")
    args = [exe, "-ic", "16", "-oc", "16", "-is", "24", "24", "-ks", "3", "3", "-ip", "1", "-a", "winograd", "-tn", "tuning",
            "-i", "2", "--strict"]
    first = _run(args, cwd=str(tmp_path))
    log = tmp_path / "gemm_log" / "mi355x_tuning_log"
    assert log.exists() and len(log.read_text().strip().splitlines()) >= 1
    assert "PASS" in first
    second = _run(args, cwd=str(tmp_path))
    assert "PASS" in second
    assert len(log.read_text().strip().splitlines()) == len(set(log.read_text().strip().splitlines()))


def test_blocked_variant_uses_the_single_kernel_engine_and_tunes(tmp_path):
    exe = _exe("conv_test")
    # 32 images of 96x96: 8192 tiles, enough blocks for the library to prefer the single-kernel engine
    base = [exe, "-ic", "16", "-oc", "24", "-is", "96", "96", "-ks", "3", "3", "-ip", "1", "-n", "32", "-i", "2",
            "-t", "16", "--strict", "-a", "winograd", "--variant", "blocked"]
    out = _run(base, cwd=str(tmp_path))
    assert "single kernel" in out and "PASS" in out
    out = _run(base + ["-tn", "tuning"], cwd=str(tmp_path))
    assert "PASS" in out and "imgb=0" in out       # the single-kernel engine was among the candidates
    # a layer outside the engine's range (8 input channels) falls back to the blocked pipeline
    out = _run([exe, "-ic", "8", "-oc", "8", "-is", "20", "20", "-ks", "3", "3", "-i", "2", "--strict", "-a", "winograd",
                "--variant", "blocked"], cwd=str(tmp_path))
    assert "single kernel" not in out and "PASS" in out


def test_layer_graph_runs_a_vgg_trunk_and_matches_the_host_chain():
    out = _run([_exe("net_test"), "-n", "2", "-is", "64", "-w", "4", "-i", "2"])
    m = re.search(r"Max relative error vs host chain: (\S+)", out)
    assert m and float(m.group(1)) <= 1e-3 and "PASS" in out
    assert "17 layers" in out


def test_layer_graph_replayed_from_a_recording_matches_the_host_chain():
    out = _run([_exe("net_test"), "-n", "1", "-is", "64", "-w", "4", "-i", "3", "--graph"])
    m = re.search(r"Max relative error vs host chain: (\S+)", out)
    assert "replay a recorded graph" in out
    assert m and float(m.group(1)) <= 1e-3 and "PASS" in out


def test_maxpool_against_numpy():
    import fastconv_amd as F
    L = F.load(0, 1 << 30)
    try:
        for (N, C, H, W) in [(2, 3, 8, 10), (1, 5, 7, 9), (3, 64, 56, 56)]:
            x = O.rng_uniform(11, (N, C, H, W))
            xd = L.upload(x)
            yd = L.alloc(N * C * (H // 2) * (W // 2) * 4)
            L.maxpool2x2(xd, yd, N, C, H, W)
            y = L.download(yd, (N, C, H // 2, W // 2))
            xe = x[:, :, :H // 2 * 2, :W // 2 * 2].reshape(N, C, H // 2, 2, W // 2, 2)
            assert np.array_equal(y, xe.max(axis=(3, 5)))
    finally:
        L.close()


def test_fill_zero_clears_exactly_its_range():
    """fc_fill_zero with 16-byte-aligned ranges (one 16-byte store per lane) and with ranges aligned
    to 4 bytes only (4-byte stores): the range reads back as zeros and its neighbours are untouched."""
    import ctypes
    import fastconv_amd as F
    L = F.load(0, 1 << 30)
    try:
        n = 1 << 16
        ones = np.ones(n, np.float32)
        buf = L.upload(ones)
        for (first, count) in [(0, n), (4, 4096), (16, 20), (1, 7), (3, 4097), (5, 1), (n - 4, 4), (n - 3, 3)]:
            L.upload_into(buf, ones)
            L.fill_zero(ctypes.c_void_p(buf.value + 4 * first), 4 * count)
            got = L.download(buf, (n,))
            expect = ones.copy()
            expect[first:first + count] = 0.0
            assert np.array_equal(got, expect), (first, count)
        with pytest.raises(F.FastConvError):
            L.fill_zero(ctypes.c_void_p(buf.value + 2), 8)          # not a 4-byte boundary
    finally:
        L.close()
