#!/usr/bin/env python3
"""Throughput of the convolution hot path on one MI355X.

A "step" is one forward pass of every conv layer of the workload (default: the
13 3x3 conv layers of VGG-16 at batch 32, Winograd F(6x6,3x3), filter transform
included) over synthetic inputs already resident in HBM.  Prints ONE JSON line:
whole-job effective GFLOP/s (direct-convolution FLOP count / wall time), the
roofline of the dominant kernel (timed with HIP events on the library's stream),
a compact `secondary` list (the batch-1 stack, the ResNet-50 layers, the three
im2col layers, each with the library's untuned choices) and a CPU baseline (the
naive direct convolution on the host cores, on a bounded sample).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--tune]

Tile shape, pipeline and algorithm per layer are the library's own untuned
choices (what the layer classes use without -tn tuning), so that a profiler run
of this same command sees the same kernels; --tune searches them per layer
first, as Tuning() of the layer classes does.  The stress workloads (batch 64
and 128) always search, and report the staged ("ZC") and the blocked layer
class side by side.
"""
import argparse
import ctypes
import json
import os
import re
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_F32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
# Measured HBM bytes per launch of the GEMM kernels (FETCH_SIZE and WRITE_SIZE of rocprofv3 --pmc, scaled by what
# the same counters read for a plain copy): a text summary under profiles/, one line per layer and tile shape.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_hbm_traffic_pmc.txt")

# (C, K, H, repeats): 3x3, stride 1, pad 1
VGG16 = [(3, 64, 224, 1), (64, 64, 224, 1), (64, 128, 112, 1), (128, 128, 112, 1), (128, 256, 56, 1),
         (256, 256, 56, 2), (256, 512, 28, 1), (512, 512, 28, 2), (512, 512, 14, 3)]
RESNET50_3X3 = [(64, 64, 56, 3), (128, 128, 28, 4), (256, 256, 14, 6), (512, 512, 7, 3)]
STRESS = [(256, 256, 56, 1), (512, 512, 28, 1), (512, 512, 14, 1)]
# (C, K, H, kernel, stride, pad, repeats): the ResNet-50 bottleneck layers
RESNET50 = [(3, 64, 224, 7, 2, 3, 1),
            (64, 64, 56, 1, 1, 0, 1), (64, 64, 56, 3, 1, 1, 3), (64, 256, 56, 1, 1, 0, 4), (256, 64, 56, 1, 1, 0, 2),
            (256, 128, 56, 1, 1, 0, 1), (128, 128, 56, 3, 2, 1, 1), (128, 128, 28, 3, 1, 1, 3),
            (128, 512, 28, 1, 1, 0, 4), (512, 128, 28, 1, 1, 0, 3), (256, 512, 56, 1, 2, 0, 1),
            (512, 256, 28, 1, 1, 0, 1), (256, 256, 28, 3, 2, 1, 1), (256, 256, 14, 3, 1, 1, 5),
            (256, 1024, 14, 1, 1, 0, 6), (1024, 256, 14, 1, 1, 0, 5), (512, 1024, 28, 1, 2, 0, 1),
            (1024, 512, 14, 1, 1, 0, 1), (512, 512, 14, 3, 2, 1, 1), (512, 512, 7, 3, 1, 1, 2),
            (512, 2048, 7, 1, 1, 0, 3), (2048, 512, 7, 1, 1, 0, 2), (1024, 2048, 14, 1, 2, 0, 1)]
IM2COL_ABC = [(256, 256, 56, 3, 1, 1, 1), (128, 256, 56, 3, 2, 1, 1), (256, 1024, 14, 1, 1, 0, 1)]


def _w(layers):
    return [(c, k, h, 3, 1, 1, r) for (c, k, h, r) in layers]


WORKLOADS = {
    # name: (layers, batch, algorithm, description)
    "vgg16_b32": (_w(VGG16), 32, "winograd", "VGG-16 conv stack, 13 layers, 3x3 s1 p1, Winograd F(6,3), batch 32"),
    "vgg16_b1": (_w(VGG16), 1, "winograd", "VGG-16 conv stack, 13 layers, 3x3 s1 p1, Winograd F(6,3), batch 1"),
    "vgg16_auto_b32": (_w(VGG16), 32, "auto", "VGG-16 conv stack, algorithm chosen per layer, batch 32"),
    "vgg16_auto_b1": (_w(VGG16), 1, "auto", "VGG-16 conv stack, algorithm chosen per layer, batch 1"),
    "resnet50_b32": (RESNET50, 32, "auto", "ResNet-50 conv layers (53 convs), algorithm chosen per layer, batch 32"),
    "resnet50_b1": (RESNET50, 1, "auto", "ResNet-50 conv layers (53 convs), algorithm chosen per layer, batch 1"),
    "resnet50_3x3_b32": (_w(RESNET50_3X3), 32, "winograd", "ResNet-50 3x3 s1 convs, Winograd F(6,3), batch 32"),
    "resnet50_3x3_b1": (_w(RESNET50_3X3), 1, "winograd", "ResNet-50 3x3 s1 convs, Winograd F(6,3), batch 1"),
    "im2col_abc_b1": (IM2COL_ABC, 1, "im2col", "3x3 256@56, 3x3 s2 128->256@56, 1x1 256->1024@14 through the implicit GEMM, batch 1"),
    "cfg1": (_w([(64, 64, 56, 1)]), 1, "winograd", "single 3x3 conv 64->64 @56, batch 1"),
    "conv3_224_b32": (_w([(3, 64, 224, 1)]), 32, "winograd", "single 3x3 conv 3->64 @224, batch 32 (VGG-16 layer 1)"),
    "conv64_224_b32": (_w([(64, 64, 224, 1)]), 32, "winograd", "single 3x3 conv 64->64 @224, batch 32 (VGG-16 layer 2)"),
    "conv256_56_b32": (_w([(256, 256, 56, 1)]), 32, "winograd", "single 3x3 conv 256->256 @56, batch 32 (VGG-16 layers 6-7)"),
    "conv512_28_b32": (_w([(512, 512, 28, 1)]), 32, "winograd", "single 3x3 conv 512->512 @28, batch 32 (VGG-16 layers 9-10)"),
    "conv512_14_b1": (_w([(512, 512, 14, 1)]), 1, "winograd", "single 3x3 conv 512->512 @14, batch 1 (VGG-16 layers 11-13): 9 tiles"),
    "igemm_3x3s2_b32": ([(128, 128, 56, 3, 2, 1, 1)], 32, "im2col", "single 3x3 stride-2 conv 128->128 @56, implicit GEMM, batch 32 (ResNet-50 conv3 entry)"),
    "igemm_1x1_b32": ([(256, 64, 56, 1, 1, 0, 1)], 32, "im2col", "single 1x1 conv 256->64 @56, implicit GEMM, batch 32 (ResNet-50 bottleneck reduce)"),
    "igemm_stem_b32": ([(3, 64, 224, 7, 2, 3, 1)], 32, "im2col", "single 7x7 stride-2 conv 3->64 @224, implicit GEMM, batch 32 (ResNet-50 stem)"),
    "igemm_512_7_b1": ([(512, 512, 7, 3, 1, 1, 1)], 1, "im2col", "single 3x3 conv 512->512 @7, implicit GEMM, batch 1 (ResNet-50 conv5): 49 pixels, reduction split over wavefronts"),
    "igemm_2048_512_7_b1": ([(2048, 512, 7, 1, 1, 0, 1)], 1, "im2col", "single 1x1 conv 2048->512 @7, implicit GEMM, batch 1 (ResNet-50 conv5 reduce): 49 pixels"),
    "stress_b64": (_w(STRESS), 64, "winograd", "VGG-16 256@56, 512@28, 512@14 at batch 64: staged (ZC) against blocked Winograd, tile shapes searched"),
    "stress_b128": (_w(STRESS), 128, "winograd", "VGG-16 256@56, 512@28, 512@14 at batch 128: staged (ZC) against blocked Winograd, tile shapes searched"),
}
# (workload, filter transform offline): compact results a default run appends
SECONDARY = (("vgg16_b1", False), ("vgg16_b1", True), ("vgg16_auto_b1", False), ("resnet50_b32", False), ("resnet50_b1", False),
             ("im2col_abc_b1", False))

ST_KT, ST_IT, ST_GEMM, ST_OT, ST_IGEMM, ST_FUSED, ST_ONEPASS = 0, 1, 2, 3, 4, 6, 7


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _offset(ptr, nbytes):
    return ctypes.c_void_p(ptr.value + nbytes)


class Layer:
    """One conv layer with its buffers resident on the device."""

    def __init__(self, L, F, N, spec, index):
        from fastconv_amd import capi
        C, K, H, ks, st, pad, repeats = spec
        self.N, self.C, self.K, self.H, self.ks, self.st, self.pad, self.repeats = N, C, K, H, ks, st, pad, repeats
        self.F = F
        self.shape = F.ConvShape(N, C, H, H, K, ks, ks, st, st, pad, pad, pad, pad)
        self.OH = self.shape.out_hw()[0]
        # the workload's inputs: uniform [-1, 1), He-normal weights, seeded per layer
        x = capi.host_uniform(2 * index + 1, (N, C, H, H))
        w = capi.host_normal(2 * index + 2, (K, C, ks, ks), float(np.sqrt(2.0 / (ks * ks * C))))
        self.x, self.w = L.upload(x), L.upload(w)
        self.y = L.alloc(4 * N * K * self.OH * self.OH)
        self.flops = self.shape.flops()
        self.algo = "winograd"        # or "im2col"
        self.plan = None              # Winograd plan
        self.U = None
        self.pipe = "staged"          # Winograd pipeline: staged, fused (GEMM + output transform) or onepass
        self.img_block = N            # fused pipeline: images per block (the blocked layer class)
        self.block_plans = None
        self.oplan = self.U2 = None   # single-kernel path: its plan and its filter layout
        self.iplan = self.Wp = self.table = self.ws = None   # implicit GEMM
        self.wino_ok = ks == 3 and st == 1
        self.candidates = None

    @property
    def fused(self):
        return self.pipe == "fused"

    def setup_onepass(self, L):
        if self.oplan is None:
            self.oplan = L.wino_onepass_plan(self.shape)
            self.U2 = L.alloc(self.oplan.U_bytes)
            L.wino_onepass_filter_transform(self.oplan, self.w, self.U2)

    def set_blocks(self, L, cfg, img_block):
        """Plans for the blocked class: the batch cut into blocks of img_block images."""
        self.img_block = img_block
        self.block_plans = None
        if img_block < self.N:
            def plan_for(n):
                s = self.F.ConvShape(n, self.C, self.H, self.H, self.K, 3, 3, 1, 1, 1, 1, 1, 1)
                return L.wino_plan(s, cfg)
            tail = self.N % img_block
            self.block_plans = (plan_for(img_block), plan_for(tail) if tail else None)

    def name(self):
        tag = "" if (self.ks, self.st) == (3, 1) else " %dx%d/s%d" % (self.ks, self.ks, self.st)
        return "%d->%d@%d%s" % (self.C, self.K, self.H, tag)

    def algorithmic(self):
        """Per-launch algorithmic work of each stage (flops for the GEMM, bytes for the transforms)."""
        T = self.plan.T
        return {
            "kt_bytes": 4.0 * self.K * self.C * (9 + 64),
            "it_bytes": 4.0 * self.N * self.C * self.H * self.H + 256.0 * self.C * T,
            "gemm_flops": 2.0 * 64 * self.K * self.C * T,
            "ot_bytes": 256.0 * self.K * T + 4.0 * self.N * self.K * self.H * self.H,
        }

    def setup_im2col(self, L, cfg):
        self.iplan = L.igemm_plan(self.shape, cfg)
        self.Wp, self.table = L.alloc(self.iplan.Wp_bytes), L.alloc(self.iplan.table_bytes)
        self.ws = L.alloc(self.iplan.ws_bytes) if self.iplan.ws_bytes else None
        L.igemm_pack_filter(self.iplan, self.w, self.Wp, self.table)


def forward(L, lay, V, M, filter_ready=False):
    """One layer pass: implicit GEMM, or Winograd staged (the ZC class: filter + input transform,
    GEMM, output transform), fused (the blocked class: GEMM + output transform in one kernel, per
    block of images) or onepass (the blocked class taken to its end: one kernel)."""
    if lay.algo == "im2col":
        L.conv_implicit_gemm(lay.iplan, lay.x, lay.Wp, lay.table, lay.y, ws=lay.ws)
    elif lay.pipe == "onepass":
        L.wino_forward_onepass(lay.oplan, lay.x, lay.w, lay.U2, lay.y, filter_ready=filter_ready)
    elif lay.fused:
        if lay.block_plans is None:
            L.wino_forward_fused(lay.plan, lay.x, lay.w, lay.U, V, lay.y, filter_ready=filter_ready)
        else:
            in_img, out_img = 4 * lay.C * lay.H * lay.H, 4 * lay.K * lay.OH * lay.OH
            full, tail = lay.block_plans
            for n0 in range(0, lay.N, lay.img_block):
                p = full if n0 + lay.img_block <= lay.N else tail
                L.wino_forward_fused(p, _offset(lay.x, n0 * in_img), lay.w, lay.U, V, _offset(lay.y, n0 * out_img),
                                     filter_ready=filter_ready or n0 > 0)
    else:
        L.wino_forward(lay.plan, lay.x, lay.w, lay.U, V, M, lay.y, filter_ready=filter_ready)


def takes_raw_filter_gemm(L, lay, filter_ready):
    """The staged pipeline multiplies straight from the 3x3 filter (no filter transform, no U) when the layer
    has few tiles and the filter is not transformed beforehand: the rule fc_wino_forward applies."""
    return (lay.algo == "winograd" and lay.pipe == "staged" and not lay.fused and not filter_ready
            and lay.block_plans is None and L.wino_prefer_raw_filter_gemm(lay.plan))


def _time(L, fn, iters):
    fn()
    L.sync()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    L.sync()
    return (time.perf_counter() - t0) / iters * 1e3


def tune_layer(L, lay, V, M, scratch_bytes, iters=3, full_search=False):
    """Whole-layer forward time of every candidate: tile shape x pipeline (x images per block for the
    blocked class when full_search).  Returns the best as (cfg, pipe, ms, img_block) and keeps the table
    of the best candidate per layer class in lay.candidates."""
    best = (None, "staged", 1e30, lay.N)
    per_class = {}
    lay.algo = "winograd"

    def note(cls, cfg, pipe, ms, ib):
        nonlocal best
        log("  candidate %s: %s cfg %s images/block %d: %.4f ms" % (lay.name(), pipe, cfg, ib, ms))
        if ms < best[2]:
            best = (cfg, pipe, ms, ib)
        if cls not in per_class or ms < per_class[cls]["ms"]:
            per_class[cls] = {"cfg": cfg, "pipe": pipe, "ms": ms, "img_block": ib}

    for cfg in L.wino_configs():
        plan = L.wino_plan(lay.shape, cfg.id)
        if plan.V_bytes > scratch_bytes[0] or plan.M_bytes > scratch_bytes[1]:
            continue
        if plan.K_pad > 2 * lay.K and cfg.bm > 32:
            continue
        lay.plan = plan
        mark = L.mark()
        lay.U = L.alloc(plan.U_bytes)
        lay.pipe = "staged"
        lay.set_blocks(L, cfg.id, lay.N)
        note("zc", cfg.id, "staged", _time(L, lambda: forward(L, lay, V, M), iters), lay.N)
        # the fused kernel has one tile shape of its own; the plan only fixes the padding it reads
        if full_search or lay.C * lay.K <= 16384:
            lay.pipe = "fused"
            blocks = [lay.N] + ([lay.N // 2, lay.N // 4] if full_search and cfg.id in (0, 3) and lay.N >= 4 else [])
            for ib in blocks:
                lay.set_blocks(L, cfg.id, ib)
                note("blocked", cfg.id, "fused", _time(L, lambda: forward(L, lay, V, M), iters), ib)
            lay.set_blocks(L, cfg.id, lay.N)
        L.release(mark)
    if full_search or lay.C <= 128:      # the whole layer in one kernel: no tile shape to choose
        try:
            lay.setup_onepass(L)
        except lay.F.FastConvError:
            pass
        else:
            lay.pipe = "onepass"
            note("blocked", None, "onepass", _time(L, lambda: forward(L, lay, V, M), iters), lay.N)
    if best[0] is None:      # the single-kernel engine won outright: the plan below still needs a tile shape
        best = (L.wino_default_config(lay.shape),) + best[1:]
    lay.candidates = per_class
    return best


def tune_im2col(L, lay, iters=3):
    best = (None, 1e30)
    lay.algo = "im2col"
    for cfg in L.igemm_configs():
        mark = L.mark()
        lay.setup_im2col(L, cfg.id)
        ms = _time(L, lambda: forward(L, lay, None, None), iters)
        L.release(mark)
        if ms < best[1]:
            best = (cfg.id, ms)
    return best


def cpu_baseline(target_seconds=3.0):
    """Naive direct convolution (the oracle's restatement of the reference's
    ConvNaiveLayer, OpenMP over images x output channels) on the VGG-16 stack,
    on a sample of about target_seconds of host time."""
    from oracle import oracle as O
    cores = O.lib().fco_num_threads()

    def run(batch):
        total_flops, total_s = 0.0, 0.0
        for (C, K, H, rep) in VGG16:
            s = O.shape(batch, C, H, H, K)
            x, w = O.make_inputs(s, seed=0)
            t0 = time.perf_counter()
            O.naive_conv_f32(s, x, w)
            dt = time.perf_counter() - t0
            total_flops += 2.0 * batch * K * C * H * H * 9 * rep
            total_s += dt * rep
        return total_flops, total_s

    fl, s1 = run(1)
    batch = int(max(1, min(32, target_seconds // max(s1, 1e-3))))
    if batch > 1:
        fl, s1 = run(batch)
    return {"value": round(fl / s1 / 1e9, 2), "unit": "GFLOP/s", "cores": cores, "kind": "port",
            "sample": "naive direct conv (restatement of the reference's ConvNaiveLayer; the reference's NEON "
                      "kernels do not build on this x86 host), VGG-16 13-layer conv stack at batch %d, %.1f s "
                      "of host time (repeated layers timed once)" % (batch, s1)}


def copy_probe(mib):
    """Plain device-to-device copy of a known size: what FETCH_SIZE / WRITE_SIZE read for it is
    the factor the counters of the other kernels are scaled by."""
    import fastconv_amd as F
    nbytes = mib << 20
    L = F.load(0, 2 * nbytes + (64 << 20))
    src, dst = L.alloc(nbytes), L.alloc(nbytes)
    L.fill_zero(src, nbytes)
    L.device_copy(dst, src, nbytes)
    L.sync()
    t0 = time.perf_counter()
    reps = 5
    for _ in range(reps):
        L.device_copy(dst, src, nbytes)
    L.sync()
    dt = (time.perf_counter() - t0) / reps
    print(json.dumps({"probe": "copy", "bytes_read": nbytes, "bytes_written": nbytes, "launches": reps + 1,
                      "ms": round(dt * 1e3, 4), "GBps_read_plus_write": round(2 * nbytes / dt / 1e9, 1)}), flush=True)
    L.close()


def measured_traffic():
    """{(kernel, N, C, K, H, ks, st, 'BMxBNxBK'): bytes per launch} parsed from the committed rocprofv3 counter
    summary; empty when the file is absent or was taken with other kernel sources than this tree's
    (`traffic` is then null)."""
    out = {}
    from fastconv_amd import provenance
    # the file names the kernel sources it was measured on: once they have changed its numbers describe other code
    if not os.path.exists(TRAFFIC_PROFILE) or not provenance.sources_current(TRAFFIC_PROFILE):
        return out
    pat = re.compile(r"^traffic kernel=(\w+) N=(\d+) C=(\d+) K=(\d+) H=(\d+) ks=(\d+) st=(\d+) tile=(\w+) "
                     r".*measured_bytes=(\d+)")
    for line in open(TRAFFIC_PROFILE):
        m = pat.match(line.strip())
        if m:
            out[(m.group(1),) + tuple(int(m.group(i)) for i in range(2, 8)) + (m.group(8),)] = int(m.group(9))
    return out


def run_workload(name, steps, warmup, o, detail=True, offline_filter=None):
    """Builds the layers of one workload on the device, times `steps` steps and returns the result fields."""
    import fastconv_amd as F
    layers_def, N, algo, desc = WORKLOADS[name]
    if getattr(o, "batch", 0):
        N = o.batch
        desc += " (batch overridden: %d)" % N
    stress = name.startswith("stress")
    tune = o.tune or stress

    # arena: activations + filters + U / packed filter per layer, one shared V and M (largest layer)
    act = sum(4 * N * (C * H * H + K * (H // st + 1) ** 2) for (C, K, H, ks, st, pad, _) in layers_def)
    tiles = lambda H: N * ((H + 5) // 6) ** 2
    wl = [(C, K, H) for (C, K, H, ks, st, pad, _) in layers_def if ks == 3 and st == 1 and algo != "im2col"]
    vmax = max([256 * (C + 32) * (tiles(H) + 256) for (C, K, H) in wl] + [256])
    mmax = max([256 * max(2 * K if K < 128 else K + 128, 128) * (tiles(H) + 256) for (C, K, H) in wl] + [256])
    umax = sum(256 * (C + 32) * (K + 256) for (C, K, H) in wl) * 2
    imax = sum(4 * (C * ks * ks + 32) * (K + 256) * 2 + 32 * 4 * N * K * (H // st + 1) ** 2 * (1 if N == 1 else 0)
               for (C, K, H, ks, st, pad, _) in layers_def) + (256 << 20)
    pool = int(act + vmax + mmax + umax + imax + (512 << 20))
    L = F.load(0, pool)
    info = L.device_info()
    log("workload %s on %s" % (name, info["arch"]))
    V, M = L.alloc(vmax), L.alloc(mmax)
    layers = [Layer(L, F, N, spec, i) for i, spec in enumerate(layers_def)]

    # algorithm, pipeline and tile shape per layer
    for lay in layers:
        want_wino = lay.wino_ok and algo in ("winograd", "auto")
        want_im2col = algo == "im2col" or not lay.wino_ok or algo == "auto"
        if algo == "winograd" and not lay.wino_ok:
            raise SystemExit("workload %s: Winograd needs 3x3 stride 1" % name)
        wres = ires = None
        if want_wino:
            if not tune:      # the library's untuned choices
                wres = (L.wino_default_config(lay.shape),
                        "onepass" if L.wino_prefer_onepass(lay.shape) else
                        "fused" if L.wino_prefer_fused(lay.shape) else "staged", 0.0, N)
            else:
                wres = tune_layer(L, lay, V, M, (vmax, mmax), full_search=stress)
        if want_im2col:
            ires = (L.igemm_default_config(lay.shape), 0.0) if not tune else tune_im2col(L, lay)
        if wres and ires:
            # -a auto: the library's rule, or the measured winner when both were timed
            use_w = L.prefer_winograd(lay.shape) if not tune else wres[2] <= ires[1]
            lay.auto_times = None if not tune else {"winograd_ms": round(wres[2], 4), "im2col_ms": round(ires[1], 4),
                                                    "rule_says": "winograd" if L.prefer_winograd(lay.shape) else "im2col"}
        else:
            use_w = wres is not None
        if use_w:
            cfg, pipe, ms, ib = wres
            if o.pipeline != "auto":
                pipe = o.pipeline
            lay.algo, lay.pipe = "winograd", pipe
            if pipe == "onepass":
                lay.setup_onepass(L)
            lay.plan = L.wino_plan(lay.shape, cfg)
            lay.U = L.alloc(lay.plan.U_bytes)
            lay.set_blocks(L, cfg, ib if pipe == "fused" else N)
            L.wino_filter_transform(lay.plan, lay.w, lay.U)
            g = L.wino_configs()[cfg]
            log("layer %s: winograd %s, tile %dx%dx%d (cfg %d)%s"
                % (lay.name(), pipe, g.bm, g.bn, g.bk, cfg,
                   " %.3f ms%s" % (ms, " (im2col %.3f ms)" % ires[1] if ires else "") if tune else ", the library's untuned choice"))
        else:
            cfg, ms = ires
            lay.algo = "im2col"
            lay.setup_im2col(L, cfg)
            g = L.igemm_configs()[cfg]
            log("layer %s: im2col, tile %dx%dx%d (cfg %d), reduction split %d over workgroups, %d over wavefronts%s"
                % (lay.name(), g.bm, g.bn, g.bk, cfg, lay.iplan.split_k, g.waves_k,
                   " %.3f ms%s" % (ms, " (winograd %.3f ms)" % wres[2] if wres else "") if tune else ", the library's untuned choice"))
    L.sync()

    filter_ready = o.offline_filter if offline_filter is None else offline_filter

    def step():
        for lay in layers:
            for _ in range(lay.repeats):
                forward(L, lay, V, M, filter_ready)

    for _ in range(warmup):
        step()
    L.sync()

    stage_events = o.stage_events
    if stage_events == "auto":
        # one more untimed step for a rough step time: brackets stay inside the timed region while
        # their own cost (about 6 us per bracketed launch) is under 2 % of the step
        t0 = time.perf_counter()
        step()
        L.sync()
        rough_us = (time.perf_counter() - t0) * 1e6
        bracketed = sum(l.repeats for l in layers if l.algo == "im2col" or l.pipe == "staged")
        stage_events = "gemm" if 6.0 * bracketed <= 0.02 * rough_us else "none"
    mask = {"all": 0xdf, "gemm": (1 << ST_GEMM) | (1 << ST_IGEMM), "none": 0}[stage_events]
    timed_step = step
    if o.graph:
        mask = 0
        L.graph_begin()
        step()
        recorded = L.graph_end()
        timed_step = lambda: L.graph_launch(recorded)
        timed_step()
        L.sync()
    L.timing(mask)
    L.timing_reset()
    t0 = time.perf_counter()
    for _ in range(steps):
        timed_step()
    L.sync()
    elapsed = time.perf_counter() - t0
    stage = [L.stage_time(i) for i in range(4)]
    fused_stage = L.stage_time(ST_FUSED)
    onepass_stage = L.stage_time(ST_ONEPASS)
    igemm_stage = L.stage_time(ST_IGEMM)
    L.timing(0)
    if stage_events != "all" and not o.timed_only:
        # the other kernels: the same steps again, untimed, every kernel bracketed
        L.timing(0xdf)
        L.timing_reset()
        for _ in range(min(steps, 5)):
            step()
        L.sync()
        detail_t = [L.stage_time(i) for i in range(4)]
        for i in (ST_KT, ST_IT, ST_OT):
            stage[i] = detail_t[i]
        fused_stage = L.stage_time(ST_FUSED)
        onepass_stage = L.stage_time(ST_ONEPASS)
        if stage_events == "none" or o.graph:
            stage[ST_GEMM] = detail_t[ST_GEMM]
            igemm_stage = L.stage_time(ST_IGEMM)
        L.timing(0)

    ms_per_step = elapsed / steps * 1e3
    # shader clock under this workload: the same steps once more, untimed, beside the library's
    # clock probe (the published MFMA peak is quoted at the maximum clock; power management runs
    # the shaders slower under fp32 MFMA load with real data)
    shader_clock = None
    if detail and not o.timed_only:
        n_probe = max(3, min(steps, 10))
        samples = 64
        sample_us = int(min(100000, max(20, ms_per_step * 1e3 * n_probe / samples)))
        step()
        step()
        L.clock_probe_begin(samples, sample_us)
        for _ in range(n_probe + 1):
            step()
        L.sync()
        mhz = L.clock_probe_end()
        shader_clock = {"nominal_mhz": info["clock_mhz"], "mean_mhz": round(sum(mhz) / len(mhz), 1),
                        "min_mhz": round(min(mhz), 1), "max_mhz": round(max(mhz), 1), "samples": len(mhz),
                        "sample_us": sample_us, "over": "%d more steps of the same workload, untimed" % n_probe}
    step_flops = sum(l.flops * l.repeats for l in layers)
    value = step_flops / (ms_per_step * 1e-3) / 1e9

    # dominant kernel: the batched GEMM. achieved = algorithmic flops of all its launches / their event time
    traffic = measured_traffic()
    wino = [l for l in layers if l.algo == "winograd"]
    staged = [l for l in wino if l.pipe == "staged"]
    gemm_flops_step = sum(l.algorithmic()["gemm_flops"] * l.repeats for l in staged)
    launches_step = max(1, sum(l.repeats for l in staged))
    roofline = {"kernel": "wino_gemm_kernel", "bound": "mfma", "achieved": None, "peak": PEAK_MFMA_F32_TFLOPS,
                "unit": "TFLOP/s", "frac": None, "traffic": None}

    def tile_name(g):
        return "%dx%dx%d" % (g.bm, g.bn, g.bk)

    if stage[ST_GEMM][1] > 0:
        gemm_ms, gemm_cnt = stage[ST_GEMM]
        ach = gemm_flops_step * (gemm_cnt / launches_step) / (gemm_ms * 1e-3) / 1e12
        keys = [("wino_gemm_kernel", N, l.C, l.K, l.H, 3, 1, tile_name(L.wino_configs()[l.plan.gemm_config]))
                for l in staged]
        if staged and all(k in traffic for k in keys):
            roofline["traffic"] = round(sum(traffic[k] * l.repeats for k, l in zip(keys, staged)) / launches_step)
            roofline["traffic_source"] = os.path.relpath(TRAFFIC_PROFILE, ROOT)
        roofline["algorithmic_bytes_per_launch_avg"] = round(
            sum(256.0 * (l.K * l.C + l.C * l.plan.T + l.K * l.plan.T) * l.repeats for l in staged) / launches_step)
        roofline.update(achieved=round(ach, 2), frac=round(ach / PEAK_MFMA_F32_TFLOPS, 4),
                        launches=gemm_cnt, avg_launch_ms=round(gemm_ms / gemm_cnt, 5),
                        flops_per_launch_avg=gemm_flops_step / launches_step)
        if shader_clock:
            # 256 CUs x 256 fp32 MFMA flops per clock: what the measured clock allows
            at_clock = info["compute_units"] * 256 * shader_clock["mean_mhz"] * 1e6 / 1e12
            roofline.update(peak_at_measured_clock=round(at_clock, 1), frac_at_measured_clock=round(ach / at_clock, 4))
    transforms = {}
    # online filter transforms of the staged and fused pipelines ride in the input transform's launch
    raw = [l for l in staged if takes_raw_filter_gemm(L, l, filter_ready)]
    if raw:
        roofline["kernel"] = "wino_gemm_kernel, wino_rawfilter_gemm_kernel (%d of %d launches per step)" % (
            sum(l.repeats for l in raw), launches_step)
    merged = [l for l in wino if l.pipe != "onepass" and l not in raw] if not filter_ready else []
    for tname, idx, key in (("input_transform", ST_IT, "it_bytes"), ("output_transform", ST_OT, "ot_bytes"),
                            ("filter_transform", ST_KT, "kt_bytes")):
        ms, cnt = stage[idx]
        if cnt > 0:
            if idx == ST_OT:
                who = staged
            elif idx == ST_IT:
                who = [l for l in wino if l.pipe != "onepass"]
            else:
                who = [l for l in wino if l not in merged and l not in raw]
            per_step = max(1, sum(l.repeats * (1 if idx != ST_IT or l.block_plans is None
                                               else -(-l.N // l.img_block)) for l in who))
            b = sum(l.algorithmic()[key] * l.repeats for l in who)
            if idx == ST_IT:
                b += sum(l.algorithmic()["kt_bytes"] * l.repeats for l in merged)
            b *= cnt / per_step
            gbs = b / (ms * 1e-3) / 1e9
            transforms[tname] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                 "frac": round(gbs / PEAK_HBM_GBS, 4), "launches": cnt}
            if idx == ST_IT and merged:
                transforms[tname]["includes"] = "filter transform (same launch)"

    if fused_stage[1] > 0:
        fl = [l for l in wino if l.fused]
        fbytes = sum((256.0 * (l.K * l.C + l.C * l.plan.T) + 4.0 * l.N * l.K * l.H * l.H) * l.repeats for l in fl)
        fflops = sum(l.algorithmic()["gemm_flops"] * l.repeats for l in fl)
        per_step_launches = sum(l.repeats * (1 if l.block_plans is None else -(-l.N // l.img_block)) for l in fl)
        k = fused_stage[1] / per_step_launches        # steps the events cover
        transforms["fused_gemm_output"] = {
            "bound": "hbm", "achieved": round(fbytes * k / (fused_stage[0] * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
            "unit": "GB/s", "frac": round(fbytes * k / (fused_stage[0] * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
            "launches": fused_stage[1], "mfma_tflops": round(fflops * k / (fused_stage[0] * 1e-3) / 1e12, 2)}

    if onepass_stage[1] > 0:
        # one kernel reads x and U and writes y: its algorithmic bytes are those three arrays
        ol = [l for l in wino if l.pipe == "onepass"]
        per_step = sum(l.repeats for l in ol)
        obytes = sum((4.0 * l.N * l.C * l.H * l.H + 256.0 * l.K * l.C + 4.0 * l.N * l.K * l.H * l.H) * l.repeats for l in ol)
        oflops = sum(l.algorithmic()["gemm_flops"] * l.repeats for l in ol)
        k = onepass_stage[1] / per_step
        gbs = obytes * k / (onepass_stage[0] * 1e-3) / 1e9
        transforms["single_kernel_conv"] = {
            "bound": "mfma", "achieved": round(oflops * k / (onepass_stage[0] * 1e-3) / 1e12, 2),
            "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s",
            "frac": round(oflops * k / (onepass_stage[0] * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4),
            "launches": onepass_stage[1], "avg_launch_ms": round(onepass_stage[0] / onepass_stage[1], 5),
            "hbm_gbs": round(gbs, 1)}
        if any(l.C <= 4 for l in ol):
            transforms["single_kernel_conv"]["note"] = "includes the launches of the small-channel kernel (no per-layer pass in this run)"

    igemm_events = None
    if igemm_stage[1] > 0:
        il = [l for l in layers if l.algo == "im2col"]
        per_step = sum(l.repeats for l in il)
        if stage_events == "none" and not o.timed_only:
            # Kernels of 10-100 us: an event pair around each launch adds 5-8 us to what it reads.  Each layer
            # is timed instead as 20 back-to-back calls between two host synchronisations (wall clock).
            L.timing(0)
            igemm_ms = sum(_time(L, lambda l=l: forward(L, l, V, M, filter_ready), 20) * l.repeats for l in il)
            igemm_stage = (igemm_ms, per_step)
            igemm_events = "20 back-to-back calls per layer after the timed region, wall clock (a split reduction's second kernel included)"
        iflops = sum(l.flops * l.repeats for l in il) * (igemm_stage[1] / per_step)
        tf = iflops / (igemm_stage[0] * 1e-3) / 1e12
        transforms["implicit_gemm"] = {"bound": "mfma", "achieved": round(tf, 2), "peak": PEAK_MFMA_F32_TFLOPS,
                                       "unit": "TFLOP/s", "frac": round(tf / PEAK_MFMA_F32_TFLOPS, 4),
                                       "launches": igemm_stage[1]}
    # the dominant kernel is the one with more time in the timed region: the implicit GEMM in the
    # ResNet-50 workloads, the staged Winograd GEMM in the VGG-16 ones
    if igemm_stage[1] > 0 and (not staged or igemm_stage[0] > stage[ST_GEMM][0]):
        wino_gemm_line = roofline if staged and stage[ST_GEMM][1] > 0 else None
        il = [l for l in layers if l.algo == "im2col"]
        def ig_key(l):
            g = L.igemm_configs()[l.iplan.config]
            if g.waves_k > 1:
                return ("igemm_wavesplit_kernel", N, l.C, l.K, l.H, l.ks, l.st, "%dx%dx%dw%d" % (g.bm, g.bn, g.bk, g.waves_k))
            return ("igemm_conv_kernel", N, l.C, l.K, l.H, l.ks, l.st, tile_name(g))
        keys = [ig_key(l) for l in il]
        tr = None
        if all(k in traffic for k in keys):
            tr = round(sum(traffic[k] * l.repeats for k, l in zip(keys, il)) / sum(l.repeats for l in il))
        n_ws = sum(l.repeats for l in il if L.igemm_configs()[l.iplan.config].waves_k > 1)
        n_all = sum(l.repeats for l in il)
        kname = ("igemm_conv_kernel" if n_ws == 0 else "igemm_wavesplit_kernel" if n_ws == n_all else
                 "igemm_wavesplit_kernel (%d of %d launches per step), igemm_conv_kernel" % (n_ws, n_all))
        roofline = dict(transforms["implicit_gemm"], kernel=kname, traffic=tr,
                        avg_launch_ms=round(igemm_stage[0] / igemm_stage[1], 5))
        if shader_clock:
            at_clock = info["compute_units"] * 256 * shader_clock["mean_mhz"] * 1e6 / 1e12
            roofline.update(peak_at_measured_clock=round(at_clock, 1),
                            frac_at_measured_clock=round(roofline["achieved"] / at_clock, 4))
        if wino_gemm_line:
            transforms["wino_gemm"] = wino_gemm_line
    elif not staged and onepass_stage[1] > 0:
        roofline = dict(transforms["single_kernel_conv"], kernel="wino_onepass_kernel", traffic=None)

    # yardstick for the HBM-bound kernels: the library's plain copy kernel (16 bytes per lane) over the
    # V and M scratch, outside the timed region
    if detail and not o.timed_only:
        nb = int(min(vmax, mmax, 1 << 30)) // 256 * 256
        if nb >= (64 << 20):
            L.device_copy(M, V, nb)
            L.sync()
            t0c = time.perf_counter()
            for _ in range(5):
                L.device_copy(M, V, nb)
            L.sync()
            gbs = 2.0 * nb * 5 / (time.perf_counter() - t0c) / 1e9
            transforms["copy_kernel"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                         "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": 2 * nb,
                                         "note": "read + write of a plain copy: what streaming kernels reach on this box"}
            # and stores alone (the library's fill kernel): the input transform writes 1.8x what it reads
            L.fill_zero(M, nb)
            L.sync()
            t0c = time.perf_counter()
            for _ in range(5):
                L.fill_zero(M, nb)
            L.sync()
            gbs = nb * 5 / (time.perf_counter() - t0c) / 1e9
            transforms["fill_kernel"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                         "frac": round(gbs / PEAK_HBM_GBS, 4), "bytes": nb,
                                         "note": "stores only: what a write-bound kernel reaches on this box"}

    def class_detail(lay, cand):
        """Time and GEMM-stage MFMA rate of one layer class's best candidate (events around every kernel)."""
        cfg = cand["cfg"] if cand["cfg"] is not None else L.wino_default_config(lay.shape)
        mark = L.mark()
        lay.pipe, lay.plan = cand["pipe"], L.wino_plan(lay.shape, cfg)
        lay.U = L.alloc(lay.plan.U_bytes)
        lay.set_blocks(L, cfg, cand["img_block"] if cand["pipe"] == "fused" else lay.N)
        L.timing(0xdf)
        L.timing_reset()
        forward(L, lay, V, M)
        L.sync()
        L.timing_reset()
        reps = 5
        for _ in range(reps):
            forward(L, lay, V, M)
        L.sync()
        st = {i: L.stage_time(i)[0] / reps for i in (ST_KT, ST_IT, ST_GEMM, ST_OT, ST_FUSED, ST_ONEPASS)}
        L.timing(0)
        L.release(mark)
        gemm_ms = st[ST_GEMM] + st[ST_FUSED] + st[ST_ONEPASS]
        g = L.wino_configs()[cfg]
        gf = lay.algorithmic()["gemm_flops"]
        row = {"ms": round(cand["ms"], 4), "gflops": round(lay.flops / (cand["ms"] * 1e-3) / 1e9, 1),
               "gemm_kernel_ms": round(gemm_ms, 4), "gemm_tflops": round(gf / (gemm_ms * 1e-3) / 1e12, 2),
               "gemm_frac_mfma": round(gf / (gemm_ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 3)}
        if cand["pipe"] == "staged":
            row.update(engine="four staged kernels, whole-layer U/V/M", tile=tile_name(g), waves="%dx%d" % (g.waves_m, g.waves_n),
                       input_tran_ms=round(st[ST_IT], 4), output_tran_ms=round(st[ST_OT], 4))
        elif cand["pipe"] == "fused":
            row.update(engine="GEMM + output transform in one kernel, no M buffer", tile="32x32x2 per wavefront, 8 wavefronts x 8 frequencies",
                       padding_of="%s plan" % tile_name(g), images_per_block=cand["img_block"],
                       input_tran_ms=round(st[ST_IT], 4))
        else:
            row.update(engine="single kernel (no V, no M)", tile="64 output channels x 16 tiles x 4 channels per chunk",
                       images_per_block=lay.N)
        return row

    # per-layer detail, outside the timed region
    per_layer = []
    L.timing(0xdf)
    for lay in ([] if (o.timed_only or not detail) else layers):
        L.timing_reset()
        reps = 5
        for _ in range(reps):
            forward(L, lay, V, M)
        L.sync()
        g = (L.igemm_configs()[lay.iplan.config] if lay.algo == "im2col" else L.wino_configs()[lay.plan.gemm_config])
        row = {"layer": lay.name(), "batch": N, "repeats": lay.repeats, "algorithm": lay.algo, "tile": tile_name(g)}
        if lay.algo == "im2col":
            ms = L.stage_time(ST_IGEMM)[0] / reps
            row.update(ms=round(ms, 4), gflops=round(lay.flops / (ms * 1e-3) / 1e9, 1), split_k=lay.iplan.split_k,
                       waves_over_reduction=g.waves_k,
                       gemm_tflops=round(lay.flops / (ms * 1e-3) / 1e12, 2),
                       gemm_frac_mfma=round(lay.flops / (ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 3))
        else:
            st = [L.stage_time(i)[0] / reps for i in range(4)]
            if lay.fused:      # one kernel does the GEMM and the output transform: listed under gemm
                st[ST_GEMM] = L.stage_time(ST_FUSED)[0] / reps
                st[ST_OT] = 0.0
            if lay.pipe == "onepass":      # one kernel does everything but the filter transform: listed under gemm
                st[ST_GEMM] = L.stage_time(ST_ONEPASS)[0] / reps
                st[ST_IT] = st[ST_OT] = 0.0
            total = sum(st)
            a = lay.algorithmic()
            raw_gemm = takes_raw_filter_gemm(L, lay, filter_ready)
            if raw_gemm:
                row["gemm_kernel"] = "wino_rawfilter_gemm_kernel (U formed in registers from the 3x3 filter)"
            row.update({
                "pipeline": lay.pipe, "ms": round(total, 4),
                "gflops": round(lay.flops / (total * 1e-3) / 1e9, 1),
                "gemm_tflops": round(a["gemm_flops"] / (st[ST_GEMM] * 1e-3) / 1e12, 2),
                "gemm_frac_mfma": round(a["gemm_flops"] / (st[ST_GEMM] * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 3),
                "input_tran_gbs": round((a["it_bytes"] + (0 if st[ST_KT] or raw_gemm else a["kt_bytes"])) / (st[ST_IT] * 1e-3) / 1e9, 0)
                if st[ST_IT] else None,
                "output_tran_gbs": round(a["ot_bytes"] / (st[ST_OT] * 1e-3) / 1e9, 0) if st[ST_OT] else None,
                "stage_ms": {"kernel_tran": round(st[ST_KT], 4), "input_tran": round(st[ST_IT], 4),
                             "gemm": round(st[ST_GEMM], 4), "output_tran": round(st[ST_OT], 4)}})
        if getattr(lay, "auto_times", None):
            row["auto"] = lay.auto_times
        per_layer.append(row)
    L.timing(0)
    if stress and detail:
        # the two layer classes side by side: best candidate of each, with the parameters it chose
        saved = [(l.pipe, l.plan, l.U, l.img_block, l.block_plans) for l in layers]
        for lay, row in zip(layers, per_layer):
            cands = lay.candidates or {}
            if "zc" in cands:
                row["zc_class"] = class_detail(lay, cands["zc"])
            if "blocked" in cands:
                row["blocked_class"] = class_detail(lay, cands["blocked"])
            if "zc" in cands and "blocked" in cands:
                row["faster_class"] = "zc" if cands["zc"]["ms"] <= cands["blocked"]["ms"] else "blocked"
        for lay, (pipe, plan, U, ib, bp) in zip(layers, saved):
            lay.pipe, lay.plan, lay.U, lay.img_block, lay.block_plans = pipe, plan, U, ib, bp

    # Two kernels answer the single-kernel calls: the MFMA one and, for layers of at most four input
    # channels, one on the vector ALUs that is bound by the stores of y.  The library books both under
    # one stage, so the two lines are taken from the per-layer pass, which times every layer by itself.
    op_rows = [(l, r) for l, r in zip(layers, per_layer) if r.get("pipeline") == "onepass"]
    if op_rows:
        def kernel_ms(rows):
            return sum(r["stage_ms"]["gemm"] * l.repeats for l, r in rows)
        big = [(l, r) for l, r in op_rows if l.C > 4]
        small = [(l, r) for l, r in op_rows if l.C <= 4]
        was_roofline = roofline.get("kernel") == "wino_onepass_kernel"
        transforms.pop("single_kernel_conv", None)
        if big:
            ms = kernel_ms(big)
            fl = sum(l.algorithmic()["gemm_flops"] * l.repeats for l, _ in big)
            by = sum((4.0 * l.N * l.C * l.H * l.H + 256.0 * l.K * l.C + 4.0 * l.N * l.K * l.H * l.H) * l.repeats for l, _ in big)
            transforms["single_kernel_conv"] = {
                "kernel": "wino_onepass_kernel", "bound": "mfma", "achieved": round(fl / (ms * 1e-3) / 1e12, 2),
                "peak": PEAK_MFMA_F32_TFLOPS, "unit": "TFLOP/s", "frac": round(fl / (ms * 1e-3) / 1e12 / PEAK_MFMA_F32_TFLOPS, 4),
                "launches_per_step": sum(l.repeats for l, _ in big), "ms_per_step": round(ms, 4),
                "hbm_gbs": round(by / (ms * 1e-3) / 1e9, 1)}
        if small:
            ms = kernel_ms(small)
            by = sum((4.0 * l.N * l.C * l.H * l.H + 1024.0 * l.K + 4.0 * l.N * l.K * l.H * l.H) * l.repeats for l, _ in small)
            transforms["small_channel_conv"] = {
                "kernel": "wino_smallc_kernel", "bound": "hbm", "achieved": round(by / (ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                "launches_per_step": sum(l.repeats for l, _ in small), "ms_per_step": round(ms, 4),
                "note": "x, the transformed filter and y once; vector ALUs only"}
        if was_roofline:
            src = transforms.get("single_kernel_conv") or transforms["small_channel_conv"]
            roofline = dict(src, traffic=None)

    roofline["events"] = ("inside the timed region" if stage_events in ("gemm", "all") and not o.graph
                          else "in the untimed steps after it")
    if str(roofline.get("kernel", "")).startswith("igemm_") and igemm_events:
        roofline["events"] = igemm_events
    out = {
        "metric": "effective GFLOP/s over the conv stack (direct-conv FLOP count / time)",
        "value": round(value, 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "description": desc, "batch": N, "algorithm": algo,
                   "per_layer": ",".join("im2col" if l.algo == "im2col" else "wino-" + l.pipe for l in layers),
                   "filter_transform": "offline" if filter_ready else "online (inside the timed region)",
                   "tuned": bool(tune), "stage_events": "none" if o.graph else stage_events,
                   "launch": "hip graph replay" if o.graph else "per-layer calls",
                   "inputs": "uniform [-1,1), He-normal weights, the library's seeded xoshiro256** stream",
                   "device": info["arch"], "compute_units": info["compute_units"], "clock_mhz": info["clock_mhz"]},
        "roofline": roofline,
        "shader_clock": shader_clock,
        "transform_rooflines": transforms,
        "layers": per_layer,
    }
    L.close()
    return out


def compact(r):
    """What the `secondary` list keeps of a workload's result."""
    rf = r["roofline"]
    return {"workload": r["config"]["workload"], "description": r["config"]["description"],
            "ms_per_step": r["ms_per_step"], "value": r["value"], "unit": r["unit"], "steps": r["steps"],
            "warmup": r["warmup"], "tuned": r["config"]["tuned"], "per_layer": r["config"]["per_layer"],
            "filter_transform": r["config"]["filter_transform"],
            "roofline": {k: rf.get(k) for k in ("kernel", "bound", "achieved", "peak", "unit", "frac", "events")}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="vgg16_b32", choices=sorted(WORKLOADS))
    ap.add_argument("--batch", type=int, default=0, metavar="N",
                    help="run the workload's layers at batch N instead of its own batch (the crossover of the two "
                         "algorithms between batch 1 and 32 is measured this way)")
    ap.add_argument("--tune", action="store_true",
                    help="search tile shape, pipeline and algorithm per layer before timing (default: the library's "
                         "untuned choices; the stress workloads always search)")
    ap.add_argument("--no-tune", action="store_true", help="(default behaviour, kept for older command lines)")
    ap.add_argument("--offline-filter", action="store_true",
                    help="transform the filters once outside the timed region")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="leave out the compact secondary workloads a default run appends")
    ap.add_argument("--stage-events", default="auto", choices=["auto", "all", "gemm", "none"],
                    help="which kernels are bracketed by events inside the timed region.  An event pair costs "
                         "5-8 us per launch: 'gemm' brackets the dominant kernel only (the other kernels are "
                         "bracketed in a few extra untimed steps), 'none' brackets nothing in the timed region "
                         "(everything comes from the untimed steps).  'auto' (default) is 'gemm' while the "
                         "brackets cost under 2 %% of a step (VGG-16 at batch 32: 9 launches in 3.5 ms), else "
                         "'none' (ResNet-50: 53 launches, 15 %% of the step; batch-1 stacks)")
    ap.add_argument("--pipeline", default="auto", choices=["auto", "staged", "fused", "onepass"],
                    help="Winograd pipeline per layer: four staged kernels, GEMM + output transform fused, the "
                         "single kernel, or what the library prefers for the layer (auto)")
    ap.add_argument("--graph", action="store_true",
                    help="record one step as a HIP graph and time replays of it (per-launch events are off; "
                         "the default times the per-layer calls the reference's driver makes)")
    ap.add_argument("--timed-only", action="store_true",
                    help="no per-layer detail pass after the timed region and no secondary workloads (every launch "
                         "of the process is then a warm-up or timed step: what a kernel trace of this command "
                         "averages over)")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="only run the plain copy kernel over MIB mebibytes (scale for the HBM traffic counters)")
    args = ap.parse_args()
    if args.copy_probe:
        return copy_probe(args.copy_probe)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the layers shard by batch with no exchange step: "
              "each GPU would hold the transformed filter and its share of the images); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    out = run_workload(args.workload, args.steps, args.warmup, args)
    if args.workload == "vgg16_b32" and not (args.no_secondary or args.timed_only):
        args.batch = 0      # the secondary workloads run at their own batch
        out["secondary"] = [compact(run_workload(w, min(args.steps, 20), args.warmup, args, detail=False,
                                                 offline_filter=off)) for (w, off) in SECONDARY]
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
