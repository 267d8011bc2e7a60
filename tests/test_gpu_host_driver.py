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
