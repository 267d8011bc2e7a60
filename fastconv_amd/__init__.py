"""MI355X (gfx950) implementation of FastConv's convolution hot path.

The product is native: HIP kernels behind a C ABI (include/fastconv_hip.h,
built into fastconv_amd/lib/libfastconv_hip.so) and the C++ layer classes and
ConvTest driver in fastconv_amd/host.  This Python package is only the ctypes
view of that ABI used by the tests and the benchmark; it holds no compute and no
CPU fallback, and raises if the library is missing or no GPU answers.
"""
from .capi import (ConvShape, FastConvError, GemmConfig, IgemmPlan, Library, WinoPlan,  # noqa: F401
                   STAGE_NAMES, build_native, load)
