"""ctypes binding of include/fastconv_hip.h (no torch, no numpy compute)."""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfastconv_hip.so")

STAGE_NAMES = ["KernelTran", "InputTran", "TensorGEMM", "OutputTran", "ImplicitGemm", "FilterPack",
               "FusedGemmOut", "OnePass"]


class FastConvError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("fastconv status %d: %s" % (status, message))
        self.status = status


class ConvShape(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("N", "C", "H", "W", "K", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr")]

    def out_hw(self):
        return ((self.H + self.pt + self.pb - self.kh) // self.sh + 1,
                (self.W + self.pl + self.pr - self.kw) // self.sw + 1)

    def flops(self):
        oh, ow = self.out_hw()
        return 2.0 * self.N * self.K * self.C * oh * ow * self.kh * self.kw


class GemmConfig(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("id", "bm", "bn", "bk", "waves_m", "waves_n", "lds_bytes", "waves_k")]


class WinoPlan(C.Structure):
    _fields_ = [("shape", ConvShape), ("OH", C.c_int), ("OW", C.c_int), ("tiles_h", C.c_int),
                ("tiles_w", C.c_int), ("T", C.c_long), ("K_pad", C.c_int), ("C_pad", C.c_int),
                ("T_pad", C.c_long), ("gemm_config", C.c_int), ("U_bytes", C.c_size_t),
                ("V_bytes", C.c_size_t), ("M_bytes", C.c_size_t)]


class IgemmPlan(C.Structure):
    _fields_ = [("shape", ConvShape), ("OH", C.c_int), ("OW", C.c_int), ("Kred", C.c_int),
                ("Kred_pad", C.c_int), ("K_pad", C.c_int), ("Npix", C.c_long), ("config", C.c_int),
                ("Wp_bytes", C.c_size_t), ("table_bytes", C.c_size_t), ("split_k", C.c_int),
                ("ws_bytes", C.c_size_t)]


class DeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 32), ("compute_units", C.c_int),
                ("clock_mhz", C.c_int), ("mem_clock_mhz", C.c_int), ("mem_bus_bits", C.c_int),
                ("total_mem", C.c_size_t), ("lds_per_block", C.c_int)]


# every symbol include/fastconv_hip.h declares: name -> (restype, argtypes)
_vp = C.c_void_p
_ABI = {
    "fc_init": (C.c_int, [C.c_int, C.POINTER(_vp)]),
    "fc_destroy": (C.c_int, [_vp]),
    "fc_get_device_info": (C.c_int, [_vp, C.POINTER(DeviceInfo)]),
    "fc_last_error": (C.c_char_p, [_vp]),
    "fc_status_string": (C.c_char_p, [C.c_int]),
    "fc_sync": (C.c_int, [_vp]),
    "fc_pool_create": (C.c_int, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "fc_pool_destroy": (C.c_int, [_vp]),
    "fc_pool_alloc": (C.c_int, [_vp, C.c_size_t, C.POINTER(_vp)]),
    "fc_pool_reset": (C.c_int, [_vp]),
    "fc_pool_mark": (C.c_int, [_vp, C.POINTER(C.c_size_t)]),
    "fc_pool_release": (C.c_int, [_vp, C.c_size_t]),
    "fc_pool_stats": (C.c_int, [_vp, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]),
    "fc_upload": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "fc_download": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "fc_fill_zero": (C.c_int, [_vp, _vp, C.c_size_t]),
    "fc_graph_begin": (C.c_int, [_vp]),
    "fc_graph_end": (C.c_int, [_vp, C.POINTER(_vp)]),
    "fc_graph_launch": (C.c_int, [_vp, _vp]),
    "fc_graph_destroy": (C.c_int, [_vp]),
    "fc_maxpool2x2": (C.c_int, [_vp, _vp, _vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "fc_device_copy": (C.c_int, [_vp, _vp, _vp, C.c_size_t]),
    "fc_host_fill_uniform": (C.c_int, [C.c_uint64, C.c_float, C.c_float, _vp, C.c_size_t]),
    "fc_host_fill_normal": (C.c_int, [C.c_uint64, C.c_float, _vp, C.c_size_t]),
    "fc_timing_enable": (C.c_int, [_vp, C.c_int]),
    "fc_timing_reset": (C.c_int, [_vp]),
    "fc_stage_time_ms": (C.c_int, [_vp, C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_long)]),
    "fc_clock_probe_begin": (C.c_int, [_vp, C.c_int, C.c_int]),
    "fc_clock_probe_end": (C.c_int, [_vp, C.POINTER(C.c_double), C.c_int, C.POINTER(C.c_int)]),
    "fc_wino_gemm_num_configs": (C.c_int, []),
    "fc_wino_gemm_get_config": (C.c_int, [C.c_int, C.POINTER(GemmConfig)]),
    "fc_wino_gemm_default_config": (C.c_int, [C.POINTER(ConvShape)]),
    "fc_igemm_default_config": (C.c_int, [C.POINTER(ConvShape)]),
    "fc_prefer_winograd": (C.c_int, [C.POINTER(ConvShape)]),
    "fc_wino_make_plan": (C.c_int, [C.POINTER(ConvShape), C.c_int, C.POINTER(WinoPlan)]),
    "fc_wino_filter_transform": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp]),
    "fc_wino_input_transform": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp]),
    "fc_wino_gemm": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp]),
    "fc_wino_gemm_raw_filter": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, C.c_int]),
    "fc_wino_raw_filter_gemm_applies": (C.c_int, [C.POINTER(WinoPlan)]),
    "fc_wino_prefer_raw_filter_gemm": (C.c_int, [C.POINTER(WinoPlan)]),
    "fc_wino_output_transform": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, C.c_int, _vp]),
    "fc_wino_filter_input_transform": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, _vp]),
    "fc_wino_gemm_output_fused": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, _vp]),
    "fc_wino_prefer_fused": (C.c_int, [C.POINTER(ConvShape)]),
    "fc_wino_make_onepass_plan": (C.c_int, [C.POINTER(ConvShape), C.POINTER(WinoPlan)]),
    "fc_wino_onepass_filter_transform": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp]),
    "fc_wino_conv_onepass": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, _vp]),
    "fc_wino_forward_onepass": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, C.c_int, _vp, _vp]),
    "fc_wino_prefer_onepass": (C.c_int, [C.POINTER(ConvShape)]),
    "fc_wino_forward_fused": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, C.c_int, _vp, _vp, _vp]),
    "fc_wino_forward": (C.c_int, [_vp, C.POINTER(WinoPlan), _vp, _vp, _vp, C.c_int, C.c_int,
                                  _vp, _vp, _vp, _vp]),
    "fc_igemm_num_configs": (C.c_int, []),
    "fc_igemm_get_config": (C.c_int, [C.c_int, C.POINTER(GemmConfig)]),
    "fc_igemm_make_plan": (C.c_int, [C.POINTER(ConvShape), C.c_int, C.POINTER(IgemmPlan)]),
    "fc_igemm_pack_filter": (C.c_int, [_vp, C.POINTER(IgemmPlan), _vp, _vp, _vp]),
    "fc_conv_implicit_gemm": (C.c_int, [_vp, C.POINTER(IgemmPlan), _vp, _vp, _vp, _vp, C.c_int, _vp, _vp]),
    "fc_conv_implicit_gemm_static": (C.c_int, [_vp, C.POINTER(IgemmPlan), _vp, _vp, _vp, _vp, C.c_int, _vp]),
}

IGEMM_STATIC_WS_BYTES = 32 << 20


def abi_symbols():
    return sorted(_ABI)


def build_native(force=True):
    """Compile the HIP library (and the C++ host driver) for gfx950."""
    cmd = ["make", "-C", _HERE, "-j8", "all"]
    if force:
        cmd.insert(3, "-B")
    subprocess.check_call(cmd)


def load_cdll():
    if not os.path.exists(LIB_PATH):
        raise FastConvError(-2, "native library %s is missing: run __graft_entry__.build() "
                            "(there is no CPU fallback)" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in _ABI.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def host_uniform(seed, shape, lo=-1.0, hi=1.0):
    """Host array of the drivers' seeded uniform stream (no GPU needed)."""
    out = np.empty(shape, np.float32)
    rc = load_cdll().fc_host_fill_uniform(seed, lo, hi, out.ctypes.data_as(_vp), out.size)
    if rc:
        raise FastConvError(rc, "fc_host_fill_uniform")
    return out


def host_normal(seed, shape, sigma):
    """Host array of the drivers' seeded normal stream (no GPU needed)."""
    out = np.empty(shape, np.float32)
    rc = load_cdll().fc_host_fill_normal(seed, sigma, out.ctypes.data_as(_vp), out.size)
    if rc:
        raise FastConvError(rc, "fc_host_fill_normal")
    return out


class Library:
    """One context + one arena on one GPU; thin, typed wrappers over the C ABI."""

    def __init__(self, device=0, pool_bytes=1 << 30):
        self.c = load_cdll()
        self.ctx = _vp()
        rc = self.c.fc_init(device, C.byref(self.ctx))
        if rc:
            raise FastConvError(rc, self.c.fc_status_string(rc).decode())
        self.pool = _vp()
        self._check(self.c.fc_pool_create(self.ctx, pool_bytes, C.byref(self.pool)))

    def close(self):
        if self.pool:
            self.c.fc_pool_destroy(self.pool)
            self.pool = None
        if self.ctx:
            self.c.fc_destroy(self.ctx)
            self.ctx = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, rc):
        if rc:
            raise FastConvError(rc, self.c.fc_last_error(self.ctx).decode())

    # ---- memory
    def alloc(self, nbytes):
        p = _vp()
        self._check(self.c.fc_pool_alloc(self.pool, nbytes, C.byref(p)))
        return p

    def mark(self):
        m = C.c_size_t()
        self._check(self.c.fc_pool_mark(self.pool, C.byref(m)))
        return m.value

    def release(self, mark):
        self._check(self.c.fc_pool_release(self.pool, mark))

    def reset_pool(self):
        self._check(self.c.fc_pool_reset(self.pool))

    def pool_stats(self):
        a, b, c_ = C.c_size_t(), C.c_size_t(), C.c_size_t()
        self._check(self.c.fc_pool_stats(self.pool, C.byref(a), C.byref(b), C.byref(c_)))
        return a.value, b.value, c_.value

    @staticmethod
    def _host_array(arr):
        """Host data as the kernels read it: C-contiguous float32 (int32 arrays pass unchanged)."""
        arr = np.asarray(arr)
        if arr.dtype != np.int32:
            arr = arr.astype(np.float32, copy=False)
        return np.ascontiguousarray(arr)

    def upload(self, arr):
        arr = self._host_array(arr)
        p = self.alloc(max(arr.nbytes, 4))
        self._check(self.c.fc_upload(self.ctx, p, arr.ctypes.data_as(_vp), arr.nbytes))
        return p

    def upload_into(self, ptr, arr):
        """Copy a host array into device memory that was allocated before."""
        arr = self._host_array(arr)
        self._check(self.c.fc_upload(self.ctx, ptr, arr.ctypes.data_as(_vp), arr.nbytes))

    def download(self, ptr, shape, dtype=np.float32):
        out = np.empty(shape, dtype)
        self._check(self.c.fc_download(self.ctx, out.ctypes.data_as(_vp), ptr, out.nbytes))
        return out

    def fill_zero(self, ptr, nbytes):
        self._check(self.c.fc_fill_zero(self.ctx, ptr, nbytes))

    def device_copy(self, dst, src, nbytes):
        self._check(self.c.fc_device_copy(self.ctx, dst, src, nbytes))

    # ---- recorded launch sequences
    def graph_begin(self):
        self._check(self.c.fc_graph_begin(self.ctx))

    def graph_end(self):
        g = _vp()
        self._check(self.c.fc_graph_end(self.ctx, C.byref(g)))
        return g

    def graph_launch(self, g):
        self._check(self.c.fc_graph_launch(self.ctx, g))

    def graph_destroy(self, g):
        rc = self.c.fc_graph_destroy(g)
        if rc:
            raise FastConvError(rc, "fc_graph_destroy")

    def maxpool2x2(self, x, y, N, Cc, H, W):
        self._check(self.c.fc_maxpool2x2(self.ctx, x, y, N, Cc, H, W))

    def sync(self):
        self._check(self.c.fc_sync(self.ctx))

    def device_info(self):
        info = DeviceInfo()
        self._check(self.c.fc_get_device_info(self.ctx, C.byref(info)))
        return {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
                "clock_mhz": info.clock_mhz, "mem_clock_mhz": info.mem_clock_mhz,
                "mem_bus_bits": info.mem_bus_bits, "total_mem": info.total_mem,
                "lds_per_block": info.lds_per_block}

    # ---- timing
    def timing(self, on):
        """on: False/0 off, True all stages, or a bit mask of (1 << stage)."""
        mask = 0xff if on is True else int(on)
        self._check(self.c.fc_timing_enable(self.ctx, mask))

    def timing_reset(self):
        self._check(self.c.fc_timing_reset(self.ctx))

    def stage_time(self, stage):
        ms, cnt = C.c_double(), C.c_long()
        self._check(self.c.fc_stage_time_ms(self.ctx, stage, C.byref(ms), C.byref(cnt)))
        return ms.value, cnt.value

    def clock_probe_begin(self, samples, sample_us):
        """Start sampling the shader clock beside whatever is enqueued next."""
        self._check(self.c.fc_clock_probe_begin(self.ctx, samples, sample_us))

    def clock_probe_end(self):
        """Wait for the probe; shader clock of every sample in MHz."""
        buf = (C.c_double * 256)()
        n = C.c_int()
        self._check(self.c.fc_clock_probe_end(self.ctx, buf, 256, C.byref(n)))
        return [buf[i] for i in range(min(n.value, 256))]

    # ---- configs / plans
    def wino_configs(self):
        out = []
        for i in range(self.c.fc_wino_gemm_num_configs()):
            g = GemmConfig()
            self.c.fc_wino_gemm_get_config(i, C.byref(g))
            out.append(g)
        return out

    def igemm_configs(self):
        out = []
        for i in range(self.c.fc_igemm_num_configs()):
            g = GemmConfig()
            self.c.fc_igemm_get_config(i, C.byref(g))
            out.append(g)
        return out

    def wino_default_config(self, shape):
        return self.c.fc_wino_gemm_default_config(C.byref(shape))

    def igemm_default_config(self, shape):
        return self.c.fc_igemm_default_config(C.byref(shape))

    def prefer_winograd(self, shape):
        """The library's rule behind `-a auto` for this layer."""
        return bool(self.c.fc_prefer_winograd(C.byref(shape)))

    def wino_plan(self, shape, config=0):
        plan = WinoPlan()
        rc = self.c.fc_wino_make_plan(C.byref(shape), config, C.byref(plan))
        if rc:
            raise FastConvError(rc, self.c.fc_status_string(rc).decode())
        return plan

    def igemm_plan(self, shape, config=0):
        plan = IgemmPlan()
        rc = self.c.fc_igemm_make_plan(C.byref(shape), config, C.byref(plan))
        if rc:
            raise FastConvError(rc, self.c.fc_status_string(rc).decode())
        return plan

    # ---- Winograd stages
    def wino_filter_transform(self, plan, w, U):
        self._check(self.c.fc_wino_filter_transform(self.ctx, C.byref(plan), w, U))

    def wino_input_transform(self, plan, x, V):
        self._check(self.c.fc_wino_input_transform(self.ctx, C.byref(plan), x, V))

    def wino_filter_input_transform(self, plan, w, U, x, V):
        self._check(self.c.fc_wino_filter_input_transform(self.ctx, C.byref(plan), w, U, x, V))

    def wino_gemm(self, plan, U, V, M):
        self._check(self.c.fc_wino_gemm(self.ctx, C.byref(plan), U, V, M))

    def wino_gemm_raw_filter(self, plan, w, V, M, freqs_per_wave=0, channel_split=0):
        self._check(self.c.fc_wino_gemm_raw_filter(self.ctx, C.byref(plan), w, V, M, int(freqs_per_wave), int(channel_split)))

    def wino_raw_filter_gemm_applies(self, plan):
        return bool(self.c.fc_wino_raw_filter_gemm_applies(C.byref(plan)))

    def wino_prefer_raw_filter_gemm(self, plan):
        return bool(self.c.fc_wino_prefer_raw_filter_gemm(C.byref(plan)))

    def wino_output_transform(self, plan, M, y, bias=None, relu=False):
        self._check(self.c.fc_wino_output_transform(self.ctx, C.byref(plan), M, bias, int(relu), y))

    def wino_gemm_output_fused(self, plan, U, V, y, bias=None, relu=False):
        self._check(self.c.fc_wino_gemm_output_fused(self.ctx, C.byref(plan), U, V, bias, int(relu), y))

    def wino_prefer_fused(self, shape):
        return bool(self.c.fc_wino_prefer_fused(C.byref(shape)))

    def wino_forward_fused(self, plan, x, w, U, V, y, bias=None, relu=False, filter_ready=False):
        self._check(self.c.fc_wino_forward_fused(self.ctx, C.byref(plan), x, w, bias, int(relu),
                                                 int(filter_ready), U, V, y))

    # ---- the whole layer in one kernel
    def wino_onepass_plan(self, shape):
        plan = WinoPlan()
        rc = self.c.fc_wino_make_onepass_plan(C.byref(shape), C.byref(plan))
        if rc:
            raise FastConvError(rc, self.c.fc_status_string(rc).decode())
        return plan

    def wino_onepass_filter_transform(self, plan, w, U):
        self._check(self.c.fc_wino_onepass_filter_transform(self.ctx, C.byref(plan), w, U))

    def wino_conv_onepass(self, plan, x, U, y, bias=None, relu=False):
        self._check(self.c.fc_wino_conv_onepass(self.ctx, C.byref(plan), x, U, bias, int(relu), y))

    def wino_forward_onepass(self, plan, x, w, U, y, bias=None, relu=False, filter_ready=False):
        self._check(self.c.fc_wino_forward_onepass(self.ctx, C.byref(plan), x, w, bias, int(relu),
                                                   int(filter_ready), U, y))

    def wino_prefer_onepass(self, shape):
        return bool(self.c.fc_wino_prefer_onepass(C.byref(shape)))

    def wino_forward(self, plan, x, w, U, V, M, y, bias=None, relu=False, filter_ready=False):
        self._check(self.c.fc_wino_forward(self.ctx, C.byref(plan), x, w, bias, int(relu),
                                           int(filter_ready), U, V, M, y))

    # ---- implicit GEMM
    def igemm_pack_filter(self, plan, w, Wp, table):
        self._check(self.c.fc_igemm_pack_filter(self.ctx, C.byref(plan), w, Wp, table))

    def conv_implicit_gemm(self, plan, x, Wp, table, y, bias=None, relu=False, ws=None):
        self._check(self.c.fc_conv_implicit_gemm(self.ctx, C.byref(plan), x, Wp, table, bias, int(relu), ws, y))

    def conv_implicit_gemm_static(self, plan, x, Wp, table, y, bias=None, relu=False):
        """As conv_implicit_gemm, with the split-reduction workspace inside the library (no allocation)."""
        self._check(self.c.fc_conv_implicit_gemm_static(self.ctx, C.byref(plan), x, Wp, table, bias, int(relu), y))

    # ---- whole-layer helpers over host arrays (tests, smoke)
    def winograd_conv_fused(self, shape, x, w, bias=None, relu=False, config=None):
        """Filter transform, input transform, then GEMM + output transform in one kernel."""
        plan = self.wino_plan(shape, self.wino_default_config(shape) if config is None else config)
        mark = self.mark()
        try:
            dx, dw = self.upload(x), self.upload(w)
            db = self.upload(bias) if bias is not None else None
            U, V = self.alloc(plan.U_bytes), self.alloc(plan.V_bytes)
            y = self.alloc(4 * shape.N * shape.K * plan.OH * plan.OW)
            self.wino_filter_transform(plan, dw, U)
            self.wino_input_transform(plan, dx, V)
            self.wino_gemm_output_fused(plan, U, V, y, db, relu)
            return self.download(y, (shape.N, shape.K, plan.OH, plan.OW))
        finally:
            self.release(mark)

    def winograd_conv_onepass(self, shape, x, w, bias=None, relu=False):
        """Filter transform into the paired layout, then the whole layer in one kernel."""
        plan = self.wino_onepass_plan(shape)
        mark = self.mark()
        try:
            dx, dw = self.upload(x), self.upload(w)
            db = self.upload(bias) if bias is not None else None
            U = self.alloc(plan.U_bytes)
            y = self.alloc(4 * shape.N * shape.K * plan.OH * plan.OW)
            self.wino_forward_onepass(plan, dx, dw, U, y, db, relu)
            return self.download(y, (shape.N, shape.K, plan.OH, plan.OW))
        finally:
            self.release(mark)

    def winograd_conv(self, shape, x, w, bias=None, relu=False, config=None, stages=False):
        plan = self.wino_plan(shape, self.wino_default_config(shape) if config is None else config)
        mark = C.c_size_t()
        self._check(self.c.fc_pool_mark(self.pool, C.byref(mark)))
        try:
            dx, dw = self.upload(x), self.upload(w)
            db = self.upload(bias) if bias is not None else None
            U, V, M = self.alloc(plan.U_bytes), self.alloc(plan.V_bytes), self.alloc(plan.M_bytes)
            y = self.alloc(4 * shape.N * shape.K * plan.OH * plan.OW)
            self.wino_forward(plan, dx, dw, U, V, M, y, db, relu)
            out = self.download(y, (shape.N, shape.K, plan.OH, plan.OW))
            if not stages:
                return out
            Uh = self.download(U, (64, plan.C_pad, plan.K_pad))
            Vh = self.download(V, (64, plan.C_pad, plan.T_pad))
            Mh = self.download(M, (64, plan.K_pad, plan.T_pad))
            return out, Uh, Vh, Mh, plan
        finally:
            self._check(self.c.fc_pool_release(self.pool, mark.value))

    def implicit_gemm_conv(self, shape, x, w, bias=None, relu=False, config=None):
        plan = self.igemm_plan(shape, self.igemm_default_config(shape) if config is None else config)
        mark = C.c_size_t()
        self._check(self.c.fc_pool_mark(self.pool, C.byref(mark)))
        try:
            dx, dw = self.upload(x), self.upload(w)
            db = self.upload(bias) if bias is not None else None
            Wp, tab = self.alloc(plan.Wp_bytes), self.alloc(plan.table_bytes)
            y = self.alloc(4 * shape.N * shape.K * plan.OH * plan.OW)
            ws = self.alloc(plan.ws_bytes) if plan.ws_bytes else None
            self.igemm_pack_filter(plan, dw, Wp, tab)
            self.conv_implicit_gemm(plan, dx, Wp, tab, y, db, relu, ws)
            return self.download(y, (shape.N, shape.K, plan.OH, plan.OW))
        finally:
            self._check(self.c.fc_pool_release(self.pool, mark.value))


def load(device=0, pool_bytes=1 << 30):
    return Library(device, pool_bytes)
