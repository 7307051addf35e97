"""R-SpMM: compressed probabilities (ACSR, row-major, row-compressed) times dense V.

Mirrors the reference's ``SPLAT/r_spmm.py``: ``rspmm_preamble`` (:128-145) and ``rspmm_launcher``
(:148-164).  The Triton kernel (:13-126) is replaced by ``splat_spmm`` (MFMA, gfx950).
"""
from __future__ import annotations

from typing import Any

import torch

import _splat_hip as _hip
from acsr_helpers import ACSRSegments, build_acsr, create_acsr, create_blocked_mask, create_windowed_mask  # noqa: F401


def rspmm_preamble(mask, output_shape: tuple[int], BLOCK_SIZE_X: int, BLOCK_SIZE_Y: int, GPU_ID: Any,
                   output_dtype: torch.dtype) -> tuple[torch.Tensor, tuple[int], int]:
    """-> (output [B, H, L, n] uninitialised, grid_dim = (ceil(n / BSX), ceil(L / BSY), B*H), T = max row nnz)."""
    dev = _hip.resolve_device(GPU_ID)
    trailing_dim_acsr = build_acsr(mask, BLOCK_SIZE_Y, dev).T
    output = torch.empty(tuple(output_shape), dtype=output_dtype, device=dev)
    grid_dim = (-(-output_shape[3] // BLOCK_SIZE_X), -(-output_shape[2] // BLOCK_SIZE_Y),
                output_shape[0] * output_shape[1])
    return (output, grid_dim, trailing_dim_acsr)


def rspmm_launcher(x: torch.Tensor, y: torch.Tensor, output: torch.Tensor,
                   dTos_linear_transformations: torch.Tensor, dTos_translations: torch.Tensor,
                   sTod_linear_transformations: torch.Tensor, sTod_translations: torch.Tensor,
                   span_loop_start: torch.Tensor, span_loop_end: torch.Tensor,
                   acsr_trailing_dim: int, nnzs: torch.Tensor, grid_dim: tuple[int],
                   BLOCK_SIZE_Y: int, BLOCK_SIZE_X: int, *, segments: ACSRSegments | None = None):
    """x = compressed probabilities [B, H, L, T]; y = V [B, H, n_keys, n]; output [B, H, L, n] written in place.
    ``span_loop_start/end`` (the reference's per-row-block key range) are accepted unchanged; the HIP
    kernel derives each workgroup's key range from the row maps themselves.
    Returns (output, sTod_linear_transformations, sTod_translations, nnzs)."""
    for name, t in (("x", x), ("y", y), ("output", output)):
        _hip.require_device_tensor(t, name)
    if x.dtype != y.dtype:
        raise _hip.SplatError("x and y must share a dtype")
    B, H, L, T = x.shape
    if T != acsr_trailing_dim:
        raise _hip.SplatError(f"x has trailing dimension {T}, expected {acsr_trailing_dim}")
    n_keys, n_out = y.shape[2], y.shape[3]
    if tuple(output.shape) != (B, H, L, n_out) or not output.is_contiguous():
        raise _hip.SplatError(f"output must be a contiguous [B, H, L, n] = {(B, H, L, n_out)} tensor")
    if not x.is_contiguous():
        x = x.contiguous()
    if y.stride(3) != 1 and n_out > 1:
        y = y.contiguous()
    segs = segments or ACSRSegments.single(dTos_linear_transformations, dTos_translations,
                                           sTod_linear_transformations, sTod_translations, nnzs, acsr_trailing_dim)
    vs = y.stride()
    dev = x.device
    arr = _hip.seg_array(segs.seg_args())
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_spmm(x.data_ptr(), y.data_ptr(), vs[0], vs[1], vs[2], output.data_ptr(), arr, len(segs),
                                   B, H, L, n_keys, n_out, T, _hip.dtype_code(x.dtype), _hip.dtype_code(output.dtype),
                                   _hip.stream_ptr(dev))
    _hip.check(rc, "splat_spmm")
    return (output, sTod_linear_transformations, sTod_translations, nnzs)
