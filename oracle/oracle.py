"""ctypes view of the CPU oracle (oracle/libfastconv_oracle.so) and, where it was
built, of the reference's own naive layers (oracle/_ref/libref_naive.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py as the checker.  The shipped package never
imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfastconv_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_naive.so")


class Shape(C.Structure):
    _fields_ = [(n, C.c_int) for n in
                ("N", "C", "H", "W", "K", "kh", "kw", "sh", "sw", "pt", "pb", "pl", "pr")]


def shape(N, Cin, H, W, K, kh=3, kw=3, sh=1, sw=1, pt=1, pb=None, pl=None, pr=None):
    pb = pt if pb is None else pb
    pl = pt if pl is None else pl
    pr = pl if pr is None else pr
    return Shape(N, Cin, H, W, K, kh, kw, sh, sw, pt, pb, pl, pr)


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference checkout exists)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"])
    if os.path.isdir("/root/reference") and (force or not os.path.exists(_REF_PATH)):
        subprocess.check_call(["make", "-C", _HERE, "ref"])


_lib = None
_ref = None
_fp = C.POINTER(C.c_float)
_dp = C.POINTER(C.c_double)


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        sp = C.POINTER(Shape)
        L.fco_out_h.argtypes = [sp]
        L.fco_out_w.argtypes = [sp]
        L.fco_wino_tiles_h.argtypes = [sp]
        L.fco_wino_tiles_w.argtypes = [sp]
        L.fco_naive_conv_f32.argtypes = [sp, _fp, _fp, _fp, C.c_int, _fp]
        L.fco_naive_conv_f64.argtypes = [sp, _fp, _fp, _fp, C.c_int, _dp]
        L.fco_wino_matrices.argtypes = [_fp, _fp, _fp]
        L.fco_wino_filter_transform.argtypes = [_fp, _fp, C.c_int, C.c_int]
        L.fco_wino_input_transform.argtypes = [sp, _fp, _fp]
        L.fco_wino_gemm.argtypes = [_fp, _fp, _fp, C.c_int, C.c_int, C.c_long]
        L.fco_wino_output_transform.argtypes = [sp, _fp, _fp, _fp]
        L.fco_wino_conv_f32.argtypes = [sp, _fp, _fp, _fp, _fp]
        L.fco_im2col.argtypes = [sp, _fp, _fp]
        L.fco_sgemm.argtypes = [C.c_int, C.c_long, C.c_int, _fp, _fp, _fp]
        L.fco_sgemm.restype = None
        L.fco_im2col_conv_f32.argtypes = [sp, _fp, _fp, _fp, _fp]
        L.fco_diff_legacy.argtypes = [_fp, _fp, C.c_long]
        L.fco_diff_legacy.restype = C.c_float
        L.fco_max_rel_err_f32.argtypes = [_fp, _dp, C.c_long]
        L.fco_max_rel_err_f32.restype = C.c_double
        L.fco_max_rel_err_f32f32.argtypes = [_fp, _fp, C.c_long]
        L.fco_max_rel_err_f32f32.restype = C.c_double
        L.fco_rng_raw.argtypes = [C.c_uint64, C.POINTER(C.c_uint64), C.c_long]
        L.fco_rng_raw.restype = None
        L.fco_rng_uniform.argtypes = [C.c_uint64, C.c_float, C.c_float, _fp, C.c_long]
        L.fco_rng_uniform.restype = None
        L.fco_rng_normal.argtypes = [C.c_uint64, C.c_float, _fp, C.c_long]
        L.fco_rng_normal.restype = None
        _lib = L
    return _lib


def ref_lib():
    """The reference's own naive layers, or None where oracle/_ref was not built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        R = C.CDLL(_REF_PATH)
        R.ref_naive_3x3s1.argtypes = [_fp, _fp, _fp] + [C.c_int] * 8
        R.ref_naive_general.argtypes = [_fp, _fp, _fp, _fp] + [C.c_int] * 12
        _ref = R
    return _ref


def _f(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_fp)


def _bias(b):
    return _f(b) if b is not None else None


def out_hw(s):
    return lib().fco_out_h(C.byref(s)), lib().fco_out_w(C.byref(s))


def tiles_hw(s):
    return lib().fco_wino_tiles_h(C.byref(s)), lib().fco_wino_tiles_w(C.byref(s))


def naive_conv_f32(s, x, w, bias=None, bias_mode=None):
    oh, ow = out_hw(s)
    y = np.empty((s.N, s.K, oh, ow), np.float32)
    mode = (0 if bias is None else 1) if bias_mode is None else bias_mode
    rc = lib().fco_naive_conv_f32(C.byref(s), _f(x), _f(w), _bias(bias), mode, _f(y))
    if rc:
        raise ValueError("fco_naive_conv_f32 rc=%d" % rc)
    return y


def naive_conv_f64(s, x, w, bias=None, bias_mode=None):
    oh, ow = out_hw(s)
    y = np.empty((s.N, s.K, oh, ow), np.float64)
    mode = (0 if bias is None else 1) if bias_mode is None else bias_mode
    rc = lib().fco_naive_conv_f64(C.byref(s), _f(x), _f(w), _bias(bias), mode,
                                  y.ctypes.data_as(_dp))
    if rc:
        raise ValueError("fco_naive_conv_f64 rc=%d" % rc)
    return y


def wino_matrices():
    BT = np.empty((8, 8), np.float32)
    G = np.empty((8, 3), np.float32)
    AT = np.empty((6, 8), np.float32)
    lib().fco_wino_matrices(_f(BT), _f(G), _f(AT))
    return BT, G, AT


def wino_filter_transform(w):
    K, Cin = w.shape[:2]
    U = np.empty((64, K, Cin), np.float32)
    rc = lib().fco_wino_filter_transform(_f(w), _f(U), K, Cin)
    if rc:
        raise ValueError("fco_wino_filter_transform rc=%d" % rc)
    return U


def wino_input_transform(s, x):
    th, tw = tiles_hw(s)
    V = np.empty((64, s.C, s.N * th * tw), np.float32)
    rc = lib().fco_wino_input_transform(C.byref(s), _f(x), _f(V))
    if rc:
        raise ValueError("fco_wino_input_transform rc=%d" % rc)
    return V


def wino_gemm(U, V):
    _, K, Cin = U.shape
    T = V.shape[2]
    M = np.empty((64, K, T), np.float32)
    rc = lib().fco_wino_gemm(_f(U), _f(V), _f(M), K, Cin, T)
    if rc:
        raise ValueError("fco_wino_gemm rc=%d" % rc)
    return M


def wino_output_transform(s, M, bias=None):
    oh, ow = out_hw(s)
    y = np.zeros((s.N, s.K, oh, ow), np.float32)
    rc = lib().fco_wino_output_transform(C.byref(s), _f(M), _bias(bias), _f(y))
    if rc:
        raise ValueError("fco_wino_output_transform rc=%d" % rc)
    return y


def wino_conv_f32(s, x, w, bias=None):
    oh, ow = out_hw(s)
    y = np.zeros((s.N, s.K, oh, ow), np.float32)
    rc = lib().fco_wino_conv_f32(C.byref(s), _f(x), _f(w), _bias(bias), _f(y))
    if rc:
        raise ValueError("fco_wino_conv_f32 rc=%d" % rc)
    return y


def im2col(s, x):
    oh, ow = out_hw(s)
    col = np.empty((s.C * s.kh * s.kw, s.N * oh * ow), np.float32)
    rc = lib().fco_im2col(C.byref(s), _f(x), _f(col))
    if rc:
        raise ValueError("fco_im2col rc=%d" % rc)
    return col


def im2col_conv_f32(s, x, w, bias=None):
    oh, ow = out_hw(s)
    y = np.empty((s.N, s.K, oh, ow), np.float32)
    rc = lib().fco_im2col_conv_f32(C.byref(s), _f(x), _f(w), _bias(bias), _f(y))
    if rc:
        raise ValueError("fco_im2col_conv_f32 rc=%d" % rc)
    return y


def diff_legacy(a, b):
    return float(lib().fco_diff_legacy(_f(a.ravel()), _f(b.ravel()), a.size))


def max_rel_err(y, ref):
    y = np.ascontiguousarray(y, np.float32).ravel()
    if ref.dtype == np.float64:
        r = np.ascontiguousarray(ref).ravel()
        return float(lib().fco_max_rel_err_f32(_f(y), r.ctypes.data_as(_dp), y.size))
    r = np.ascontiguousarray(ref, np.float32).ravel()
    return float(lib().fco_max_rel_err_f32f32(_f(y), _f(r), y.size))


def rng_raw(seed, n):
    out = np.empty(n, np.uint64)
    lib().fco_rng_raw(seed, out.ctypes.data_as(C.POINTER(C.c_uint64)), n)
    return out


def rng_uniform(seed, shape_, lo=-1.0, hi=1.0):
    out = np.empty(shape_, np.float32)
    lib().fco_rng_uniform(seed, lo, hi, _f(out), out.size)
    return out


def rng_normal(seed, shape_, sigma):
    out = np.empty(shape_, np.float32)
    lib().fco_rng_normal(seed, sigma, _f(out), out.size)
    return out


def make_inputs(s, seed=0):
    """The workload definition: input uniform[-1,1), He-normal weights
    sigma = sqrt(2 / (kh*kw*C)), both from the seeded xoshiro256** stream."""
    x = rng_uniform(seed * 2 + 1, (s.N, s.C, s.H, s.W))
    w = rng_normal(seed * 2 + 2, (s.K, s.C, s.kh, s.kw),
                   float(np.sqrt(2.0 / (s.kh * s.kw * s.C))))
    return x, w


def ref_naive_3x3s1(s, x, w):
    """The reference's convLayer/naiveConv.h layer, looped over the batch."""
    R = ref_lib()
    oh, ow = out_hw(s)
    y = np.empty((s.N, s.K, oh, ow), np.float32)
    for n in range(s.N):
        R.ref_naive_3x3s1(_f(x[n]), _f(w), _f(y[n]), s.C, s.H, s.W, s.K,
                          s.pl, s.pr, s.pt, s.pb)
    return y


def ref_naive_general(s, x, w, bias_elems=None):
    """The reference's convLayer/naiveConv_wudu.h layer, looped over the batch."""
    R = ref_lib()
    oh, ow = out_hw(s)
    y = np.empty((s.N, s.K, oh, ow), np.float32)
    for n in range(s.N):
        R.ref_naive_general(_f(x[n]), _f(w), _bias(bias_elems), _f(y[n]), s.C, s.H, s.W, s.K,
                            s.kh, s.kw, s.sh, s.sw, s.pl, s.pr, s.pt, s.pb)
    return y
