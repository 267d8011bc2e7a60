"""Host-side C++ logic (memory pools over the arena, tuning log, algorithm choice,
layer geometry, the driver's input generator): built with g++ and run here, no GPU."""
import os
import subprocess

import numpy as np

from oracle import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "fastconv_amd")


def _build():
    subprocess.check_call(["make", "-C", PKG, "-s", "hosttest"])
    return os.path.join(PKG, "bin", "test_host")


def test_host_unit_tests_pass():
    exe = _build()
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all host tests passed" in r.stdout


def test_host_unit_tests_pass_under_address_and_undefined_behaviour_sanitizers():
    """The pools, the range allocator, the tuning log and the naive layer are pointer-heavy host code:
    the same unit tests, built with -fsanitize=address,undefined (host code only)."""
    subprocess.check_call(["make", "-C", PKG, "-s", "hosttest-san"])
    env = dict(os.environ, ASAN_OPTIONS="verify_asan_link_order=0:abort_on_error=1", UBSAN_OPTIONS="halt_on_error=1")
    r = subprocess.run([os.path.join(PKG, "bin", "test_host_san")], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all host tests passed" in r.stdout
    assert "ERROR: AddressSanitizer" not in r.stderr and "runtime error" not in r.stderr


def test_driver_generator_matches_oracle_generator_bit_for_bit():
    exe = _build()
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120,
                       env=dict(os.environ, FASTCONV_DUMP_RNG="1"))
    assert r.returncode == 0
    u = [float.fromhex(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("U ")]
    g = [float.fromhex(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("G ")]
    assert np.array_equal(np.array(u, np.float32), O.rng_uniform(7, (1000,))[:8])
    assert np.array_equal(np.array(g, np.float32), O.rng_normal(7, (1001,), 0.5)[:8])


def test_host_naive_layer_reproduces_the_reference_naive_layers_bit_for_bit(tmp_path):
    """host/convLayer/naiveConv.h is the checker of conv_test and net_test: on every stored
    case of the reference's own ConvNaiveLayers (tests/golden/naive_ref_vectors.npz) it
    must give the same bits."""
    exe = _build()
    z = np.load(os.path.join(ROOT, "tests", "golden", "naive_ref_vectors.npz"))
    names = sorted({k.split("/")[0] for k in z.files})
    assert len(names) >= 10
    for name in names:
        has_bias = name + "/bias_elems" in z.files
        src, dst = tmp_path / (name + ".in"), tmp_path / (name + ".out")
        with open(src, "wb") as f:
            f.write(z[name + "/shape"].astype(np.int32).tobytes())
            f.write(np.int32(1 if has_bias else 0).tobytes())
            f.write(np.ascontiguousarray(z[name + "/x"], np.float32).tobytes())
            f.write(np.ascontiguousarray(z[name + "/w"], np.float32).tobytes())
            if has_bias:
                f.write(np.ascontiguousarray(z[name + "/bias_elems"], np.float32).tobytes())
        r = subprocess.run([exe, "--naive", str(src), str(dst)], capture_output=True, text=True, timeout=60)
        assert r.returncode == 0, (name, r.stderr)
        y = np.fromfile(dst, np.float32).reshape(z[name + "/y"].shape)
        assert np.array_equal(y, z[name + "/y"]), name


def test_driver_refuses_to_run_without_a_gpu_or_reports_results():
    """conv_test has no CPU compute path: without a GPU it must stop with an error."""
    exe = os.path.join(PKG, "bin", "conv_test")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", PKG, "-s", "host"])
    r = subprocess.run([exe, "-ic", "4", "-oc", "4", "-is", "8", "8", "-ks", "3", "3", "-i", "1"],
                       capture_output=True, text=True, timeout=120)
    if r.returncode != 0:
        assert "no CPU path" in r.stderr
    else:
        assert "PASS" in r.stdout


def test_driver_argument_errors():
    exe = os.path.join(PKG, "bin", "conv_test")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", PKG, "-s", "host"])
    for args, msg in [([], "input channels is not specified"),
                      (["-ic", "4"], "output channels is not specified"),
                      (["-ic", "4", "-oc", "4", "-ks", "3", "3"], "input size is not specified"),
                      (["-ic", "0"], "positive value expected"),
                      (["-ic", "x"], "can not parse"),
                      (["-a", "fft"], "invalid convolution algorithm"),
                      (["--frobnicate"], "unknown argument")]:
        r = subprocess.run([exe] + args, capture_output=True, text=True, timeout=60)
        assert r.returncode != 0 and msg in r.stderr, (args, r.stderr)
