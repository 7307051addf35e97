"""ctypes binding of libsplat_hip.so (C ABI declared in include/splat_hip.h).

The library is the only compute path of this package: if it cannot be loaded, or no HIP device is
present, every operator raises -- there is no host fallback.
"""
from __future__ import annotations

import ctypes
import os
from typing import Any, Sequence

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# SPLAT_HIP_LIB selects another build of the same library (e.g. an instrumented one)
LIB_PATH = os.environ.get("SPLAT_HIP_LIB") or os.path.normpath(os.path.join(_HERE, "..", "lib", "libsplat_hip.so"))

SPLAT_F32, SPLAT_F16, SPLAT_BF16 = 0, 1, 2
MAX_SEGMENTS = 4
MASK_BLOCKED, MASK_WINDOWED, MASK_CAUSAL_WINDOWED, MASK_DILATED, MASK_STRIDED_LOCAL, MASK_STRIDED_FAR = range(6)
MASK_TRANSPOSED = 8  # flag or-ed onto a pattern: its transpose
STATIC_PLAN_BYTES = 4 << 20  # SPLAT_STATIC_PLAN_BYTES: the plan buffer built into the library for splat_attention_fwd_noalloc

_DTYPES = {torch.float32: SPLAT_F32, torch.float16: SPLAT_F16, torch.bfloat16: SPLAT_BF16}


class SplatError(RuntimeError):
    """A libsplat_hip entry point returned a non-zero code."""


class AcsrSeg(ctypes.Structure):
    _fields_ = [("dTos_lin", ctypes.c_void_p), ("dTos_trans", ctypes.c_void_p), ("sTod_lin", ctypes.c_void_p),
                ("sTod_trans", ctypes.c_void_p), ("nnz", ctypes.c_void_p), ("first_col", ctypes.c_void_p),
                ("slot_offset", ctypes.c_int32), ("row_stride_hint", ctypes.c_int32)]


_lib = None

_i32, _i64, _f32, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
_SIGNATURES = {
    "splat_version": (ctypes.c_int, []),
    "splat_last_error": (ctypes.c_char_p, []),
    "splat_acsr_build": (ctypes.c_int, [_vp, _i64, _i64, _i64, _i32] + [_vp] * 10 + [_vp]),
    "splat_mask_generate": (ctypes.c_int, [_vp, _i64, _i64, _i64, _i32, _i64, _i64, _vp]),
    "splat_acsr_build_pattern": (ctypes.c_int, [_i32, _i64, _i64, _i64, _i32] + [_vp] * 10 + [_vp]),
    "splat_sddmm": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), _i32,
                                   _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _vp]),
    "splat_sddmm_probs": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), _i32,
                                         _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _vp, _vp]),
    "splat_sddmm_planned": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), _i32,
                                           _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _i32, _vp, _vp, _i64, _vp]),
    "splat_softmax": (ctypes.c_int, [_vp, _vp, ctypes.POINTER(AcsrSeg), _i32, _i64, _i32, _i32, _i32, _i32, _vp]),
    "splat_spmm": (ctypes.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32, _i32,
                                  _i32, _i32, _i32, _i32, _vp]),
    "splat_spmm_planned": (ctypes.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32, _i32,
                                          _i32, _i32, _i32, _i32, _vp, _i64, _vp]),
    "splat_attention_fwd": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp,
                                           _i64, _i64, _i64, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32, _i32, _f32,
                                           _i32, _vp]),
    "splat_attention_fwd_noalloc": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _vp,
                                                   _i64, _i64, _i64, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32, _i32,
                                                   _f32, _i32, _vp]),
    "splat_transpose_keys": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i32, _i32, _i32, _i32, _i32, _vp]),
    "splat_softmax_bwd": (ctypes.c_int, [_vp, _vp, _vp, ctypes.POINTER(AcsrSeg), _i32, _i64, _i32, _i32, _f32, _i32, _vp]),
    "splat_spmm_t": (ctypes.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), ctypes.POINTER(AcsrSeg), _i32, _i32,
                                   _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "splat_spmm_t_planned": (ctypes.c_int, [_vp, _vp, _i64, _i64, _i64, _vp, ctypes.POINTER(AcsrSeg), ctypes.POINTER(AcsrSeg), _i32,
                                            _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _i64, _vp]),
    "splat_compressed_transpose": (ctypes.c_int, [_vp, _vp, ctypes.POINTER(AcsrSeg), ctypes.POINTER(AcsrSeg), _i32, _i64, _i32,
                                                  _i32, _i32, _i32, _i32, _vp]),
    "splat_attention_plan_bytes": (ctypes.c_int64, [ctypes.POINTER(AcsrSeg), _i32, _i32]),
    "splat_attention_plan": (ctypes.c_int, [ctypes.POINTER(AcsrSeg), _i32, _i32, _vp, _i64, _vp]),
    "splat_attention_fwd_planned": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
                                                   _vp, _i64, _i64, _i64, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32,
                                                   _i32, _f32, _i32, _vp, _i64, _vp]),
    "splat_attention_fwd_stats": (ctypes.c_int, [_vp, _i64, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64, _i64, _i64,
                                                 _vp, _i64, _i64, _i64, ctypes.POINTER(AcsrSeg), _i32, _i32, _i32, _i32,
                                                 _i32, _f32, _i32, _vp, _i64, _vp, _vp]),
    "splat_attention_bwd": (ctypes.c_int, [_vp, _i64, _i64, _i64] * 5 + [_vp] * 5 +
                            [ctypes.POINTER(AcsrSeg), _i32, _vp, _i64] * 2 + [_i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "splat_attention_bwd_keys": (ctypes.c_int, [_vp, _i64, _i64, _i64] * 4 + [_vp] * 5 +
                                 [ctypes.POINTER(AcsrSeg), _i32, _vp, _i64] + [_i32, _i32, _i32, _i32, _i32, _f32, _i32] +
                                 [_vp, _vp, _i32, _vp]),
}
EXPORTS = tuple(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load (once) and return the shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise SplatError(f"{LIB_PATH} is missing: build it with `python triton-fun_amd/build.py` "
                             "(there is no fallback path)")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().splat_last_error().decode("utf-8", "replace")
        raise SplatError(f"{what} failed (code {rc}): {msg}")


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPES[dt]
    except KeyError:
        raise SplatError(f"unsupported dtype {dt}: use float32, float16 or bfloat16") from None


def resolve_device(GPU_ID: Any) -> torch.device:
    """GPU_ID as the reference passes it to ``.to()``: an int ordinal, a device string or a torch.device.
    Only HIP devices are accepted; the kernels have no host implementation."""
    dev = torch.device("cuda", GPU_ID) if isinstance(GPU_ID, int) else torch.device(GPU_ID)
    if dev.type != "cuda":
        raise SplatError(f"GPU_ID={GPU_ID!r}: this implementation runs on a HIP device only (no CPU path)")
    if not torch.cuda.is_available():
        raise SplatError("no HIP device is available")
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    return dev


def stream_ptr(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_device_tensor(t: torch.Tensor, name: str) -> None:
    if not isinstance(t, torch.Tensor) or t.device.type != "cuda":
        raise SplatError(f"{name} must be a tensor on a HIP device")


def seg_array(segments: Sequence[tuple], rows: int, trailing_dim: int | None = None) -> Any:
    """segments: (dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnzs, first_col | None, slot_offset); the row-stride
    hint is read from the attribute ``splat_row_stride`` of sTod_trans when the builder attached one.

    ``rows`` is the number of mask rows the launch will index the arrays with (the C ABI takes bare pointers, so this
    is the only place where their length can be checked); ``trailing_dim``, when the launch has a compressed buffer,
    the number of slots of its rows, which every segment's offset must lie inside."""
    if not 1 <= len(segments) <= MAX_SEGMENTS:
        raise SplatError(f"between 1 and {MAX_SEGMENTS} ACSR segments are supported (got {len(segments)})")
    arr = (AcsrSeg * len(segments))()
    for i, (a, b, c, d, n, fc, off) in enumerate(segments):
        for name, t in (("dTos_lin", a), ("dTos_trans", b), ("sTod_lin", c), ("sTod_trans", d), ("nnzs", n)):
            require_device_tensor(t, name)
            if t.dtype != torch.float32 or not t.is_contiguous():
                raise SplatError(f"{name} must be a contiguous float32 tensor")
            if t.numel() < rows:
                raise SplatError(f"{name} of segment {i} has {t.numel()} entries, the launch has {rows} rows: the ACSR "
                                 "was built for another mask")
        if fc is not None:
            require_device_tensor(fc, "first_col")
            if fc.dtype != torch.int32 or not fc.is_contiguous() or fc.numel() < rows:
                raise SplatError(f"first_col of segment {i} must be a contiguous int32 tensor with at least {rows} entries")
        if trailing_dim is not None and not 0 <= int(off) < max(int(trailing_dim), 1):
            raise SplatError(f"segment {i} starts at slot {off}, outside the compressed rows' {trailing_dim} slots")
        arr[i].dTos_lin, arr[i].dTos_trans = a.data_ptr(), b.data_ptr()
        arr[i].sTod_lin, arr[i].sTod_trans, arr[i].nnz = c.data_ptr(), d.data_ptr(), n.data_ptr()
        arr[i].first_col = fc.data_ptr() if fc is not None else None
        arr[i].slot_offset = int(off)
        arr[i].row_stride_hint = int(getattr(d, "splat_row_stride", 1))
    return arr
