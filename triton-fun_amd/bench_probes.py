"""ctypes binding of libsplat_bench.so (C ABI declared in include/splat_bench.h): the two measurement aids bench.py
quotes the kernels against.  Not part of the operator package: nothing under SPLAT/ imports it."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("SPLAT_BENCH_LIB") or os.path.join(_HERE, "lib", "libsplat_bench.so")

_i32, _i64, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
_SIGNATURES = {
    "splat_bench_version": (ctypes.c_int, []),
    "splat_bench_last_error": (ctypes.c_char_p, []),
    "splat_bench_stream_copy": (ctypes.c_int, [_vp, _vp, _i64, _vp]),
    "splat_bench_mfma_lds_probe": (ctypes.c_int, [_vp, _i64, _vp, _i64, _i32, _i32, _i32, _vp]),
    "splat_bench_mfma_lds_probe_flops": (ctypes.c_int64, [_i32, _i32, _i32]),
    "splat_bench_softmax_loop_probe": (ctypes.c_int, [_vp, _i64, _vp, _i64, _i32, _i32, _i32, _i32, _vp]),
    "splat_bench_softmax_loop_probe_flops": (ctypes.c_int64, [_i32, _i32]),
}
EXPORTS = tuple(_SIGNATURES)
PROBE_SHAPES = {0: "32x32x16, 32 rows per wavefront, 2 wavefronts per SIMD",
                1: "32x32x16, 64 rows per wavefront, 1 wavefront per SIMD",
                2: "16x16x32, 16 rows per wavefront, 4 wavefronts per SIMD"}
PROBE_THREADS = {0: 256, 1: 256, 2: 512}
SOFTMAX_LOOP_SHAPES = {0: "32x32x16, 32 rows per wavefront, 3 wavefronts per SIMD",
                       1: "16x16x32, 16 rows per wavefront, 6 wavefronts per SIMD"}
SOFTMAX_LOOP_THREADS = {0: 256, 1: 512}

_lib = None


def lib() -> ctypes.CDLL:
    """Load (once) and return the library; raises if it has not been built (``python triton-fun_amd/build.py``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python triton-fun_amd/build.py`")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed (code {rc}): {lib().splat_bench_last_error().decode('utf-8', 'replace')}")
