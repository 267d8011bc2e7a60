"""The C-ABI library loads and exports exactly what include/fastconv_hip.h
declares.  No compute is called here (this file runs without a GPU)."""
import ctypes as C
import os
import re

from fastconv_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "fastconv_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fc_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_name_the_same_symbols():
    assert _declared() == capi.abi_symbols()


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(capi.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name


def test_status_strings_and_config_tables_need_no_gpu():
    lib = capi.load_cdll()
    assert lib.fc_status_string(0) == b"ok"
    assert lib.fc_status_string(-4) == b"out of device memory"
    n = lib.fc_wino_gemm_num_configs()
    assert n >= 4
    seen = set()
    for i in range(n):
        g = capi.GemmConfig()
        assert lib.fc_wino_gemm_get_config(i, C.byref(g)) == 0
        assert g.id == i and g.bm % 32 == 0 and g.bn % 32 == 0 and g.bk % 2 == 0
        assert g.lds_bytes == 2 * g.bk * (g.bm + g.bn) * 4 <= 64 * 1024
        seen.add((g.bm, g.bn, g.bk, g.waves_m, g.waves_n))
    assert len(seen) == n
    assert lib.fc_wino_gemm_get_config(n, C.byref(capi.GemmConfig())) == -1
    for i in range(lib.fc_igemm_num_configs()):
        g = capi.GemmConfig()
        assert lib.fc_igemm_get_config(i, C.byref(g)) == 0
        assert (64 * g.waves_m * g.waves_n) % g.bn == 0


def test_plans_are_pure_host_arithmetic():
    lib = capi.load_cdll()
    s = capi.ConvShape(32, 256, 56, 56, 256, 3, 3, 1, 1, 1, 1, 1, 1)
    p = capi.WinoPlan()
    assert lib.fc_wino_make_plan(C.byref(s), 0, C.byref(p)) == 0
    assert (p.OH, p.OW, p.tiles_h, p.tiles_w, p.T) == (56, 56, 10, 10, 3200)
    assert (p.K_pad, p.C_pad, p.T_pad) == (256, 256, 3200)
    assert p.V_bytes == 64 * 256 * 3200 * 4 and p.M_bytes == p.V_bytes and p.U_bytes == 64 * 256 * 256 * 4
    # winoF63ZC/winoF63ZC.cpp:336-338: ceil(OH/6) tiles, also when OH is not a multiple of 6
    s2 = capi.ConvShape(1, 3, 7, 9, 5, 3, 3, 1, 1, 1, 1, 1, 1)
    assert lib.fc_wino_make_plan(C.byref(s2), 4, C.byref(p)) == 0
    assert (p.tiles_h, p.tiles_w, p.T, p.K_pad, p.C_pad, p.T_pad) == (2, 2, 4, 32, 16, 32)
    # Winograd is 3x3 stride 1 only
    s3 = capi.ConvShape(1, 3, 8, 8, 5, 3, 3, 2, 2, 1, 1, 1, 1)
    assert lib.fc_wino_make_plan(C.byref(s3), 0, C.byref(p)) == -1
    q = capi.IgemmPlan()
    assert lib.fc_igemm_make_plan(C.byref(s3), 0, C.byref(q)) == 0
    assert (q.OH, q.OW, q.Kred, q.Npix) == (4, 4, 27, 16)
    assert q.Kred_pad == 32 and q.K_pad == 128
    assert q.split_k == 1 and q.ws_bytes == 0              # 2 stages: too short to split
    # a batch-1 layer with 8 workgroups of output and a long reduction is split, with workspace
    s4 = capi.ConvShape(1, 2048, 7, 7, 512, 1, 1, 1, 1, 0, 0, 0, 0)
    assert lib.fc_igemm_make_plan(C.byref(s4), 0, C.byref(q)) == 0
    assert q.split_k > 1 and q.ws_bytes == 4 * q.split_k * 512 * 49
    assert (q.Kred_pad // 16) >= 4 * q.split_k


def test_winograd_width_limit_is_part_of_the_plan_and_of_the_auto_rule():
    lib = capi.load_cdll()
    p = capi.WinoPlan()
    ok = capi.ConvShape(8, 64, 9, 1020, 64, 3, 3, 1, 1, 1, 1, 1, 1)
    wide = capi.ConvShape(8, 64, 9, 1021, 64, 3, 3, 1, 1, 1, 1, 1, 1)
    assert lib.fc_wino_make_plan(C.byref(ok), 0, C.byref(p)) == 0 and p.tiles_w == 170
    assert lib.fc_wino_make_plan(C.byref(wide), 0, C.byref(p)) == -6
    assert lib.fc_prefer_winograd(C.byref(ok)) == 1 and lib.fc_prefer_winograd(C.byref(wide)) == 0
    strided = capi.ConvShape(8, 64, 56, 56, 64, 3, 3, 2, 2, 1, 1, 1, 1)
    assert lib.fc_prefer_winograd(C.byref(strided)) == 0
    few_channels = capi.ConvShape(32, 3, 224, 224, 64, 3, 3, 1, 1, 1, 1, 1, 1)
    little_work = capi.ConvShape(1, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1, 1, 1)
    assert lib.fc_prefer_winograd(C.byref(few_channels)) == 0 and lib.fc_prefer_winograd(C.byref(little_work)) == 0


def test_library_generator_is_the_oracle_generator():
    import numpy as np
    from oracle import oracle as O
    assert np.array_equal(capi.host_uniform(7, (3, 333)), O.rng_uniform(7, (3, 333)))
    assert np.array_equal(capi.host_normal(9, (1001,), 0.25), O.rng_normal(9, (1001,), 0.25))


def test_no_gpu_means_a_loud_error_not_a_fallback():
    import pytest
    lib = capi.load_cdll()
    ctx = C.c_void_p()
    rc = lib.fc_init(0, C.byref(ctx))
    if rc == 0:                       # a GPU is present: nothing to check here
        lib.fc_destroy(ctx)
        return
    assert rc == -2 and not ctx.value
    with pytest.raises(capi.FastConvError):
        capi.Library(0)


def test_struct_layouts_match_the_header(tmp_path):
    """sizeof and every field offset of the ctypes structures against what a C compiler makes of
    include/fastconv_hip.h."""
    import subprocess
    structs = {"fc_conv_shape": capi.ConvShape, "fc_gemm_config": capi.GemmConfig, "fc_wino_plan": capi.WinoPlan,
               "fc_igemm_plan": capi.IgemmPlan, "fc_device_info": capi.DeviceInfo}
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "fastconv_hip.h"', 'int main(void) {']
    for cname, ct in structs.items():
        lines.append('printf("%s sizeof %%zu\\n", sizeof(%s));' % (cname, cname))
        for fname, _ in ct._fields_:
            lines.append('printf("%s %s %%zu\\n", offsetof(%s, %s));' % (cname, fname, cname, fname))
    lines += ['return 0;', '}']
    src, exe = tmp_path / "layout.c", tmp_path / "layout"
    src.write_text("\n".join(lines))
    subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    seen = 0
    for line in subprocess.check_output([str(exe)], text=True).splitlines():
        cname, field, value = line.split()
        ct = structs[cname]
        if field == "sizeof":
            assert C.sizeof(ct) == int(value), cname
        else:
            assert getattr(ct, field).offset == int(value), (cname, field)
        seen += 1
    assert seen == sum(len(ct._fields_) + 1 for ct in structs.values())
    assert len(capi.STAGE_NAMES) == 8       # FC_STAGE_COUNT


def test_bench_reads_measured_traffic_from_the_committed_profile():
    """bench.py takes roofline.traffic from profiles/gemm_hbm_traffic_pmc.txt: every GEMM launch of the
    default workload (library choices) must be in it, with a plausible ratio to the algorithmic bytes."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("bench", os.path.join(ROOT, "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    table = bench.measured_traffic()
    assert table, "profiles/gemm_hbm_traffic_pmc.txt has no traffic lines"
    lib = capi.load_cdll()
    layers, N, algo, _ = bench.WORKLOADS["vgg16_b32"]
    seen = 0
    for (Cc, K, H, ks, st, pad, rep) in layers:
        s = capi.ConvShape(N, Cc, H, H, K, ks, ks, st, st, pad, pad, pad, pad)
        if lib.fc_wino_prefer_onepass(C.byref(s)) or lib.fc_wino_prefer_fused(C.byref(s)):
            continue                                   # no staged GEMM launch for this layer
        g = capi.GemmConfig()
        assert lib.fc_wino_gemm_get_config(lib.fc_wino_gemm_default_config(C.byref(s)), C.byref(g)) == 0
        key = ("wino_gemm_kernel", N, Cc, K, H, 3, 1, "%dx%dx%d" % (g.bm, g.bn, g.bk))
        assert key in table, key
        T = N * ((H + 5) // 6) ** 2
        algorithmic = 256.0 * (K * Cc + Cc * T + K * T)
        assert 0.95 <= table[key] / algorithmic <= 1.25, (key, table[key] / algorithmic)
        seen += 1
    assert seen >= 5


def test_bench_refuses_more_than_one_gpu_with_a_message():
    """bench.py --gpus N with N above 1 exits before touching the GPU and says why."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
