"""R-SpMM: compressed probabilities (ACSR, row-major, row-compressed) times dense V.

Mirrors the reference's ``SPLAT/r_spmm.py``: ``rspmm_preamble`` (:128-145) and ``rspmm_launcher``
(:148-164).  The Triton kernel (:13-126) is replaced by ``splat_spmm`` (MFMA, gfx950).  The module's self-check
(``is_correct`` :166-216, ``test`` :219-261) keeps its names, signatures and acceptance rule.
"""
from __future__ import annotations

from typing import Any

import torch

import _splat_hip as _hip
from acsr_helpers import ACSRSegments, build_acsr, create_acsr, create_blocked_mask, create_windowed_mask  # noqa: F401
from r_sddmm import live_slot_columns


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
                   BLOCK_SIZE_Y: int, BLOCK_SIZE_X: int, *, segments: ACSRSegments | None = None,
                   plan: torch.Tensor | None | bool = None):
    """x = compressed probabilities [B, H, L, T]; y = V [B, H, n_keys, n]; output [B, H, L, n] written in place.
    ``span_loop_start/end`` (the reference's per-row-block key range) are accepted unchanged; the HIP
    kernel derives each workgroup's key range from the row maps themselves.
    ``plan``: the mask's plan table (``ACSRSegments.plan``), which selects the kernels that start from it where the library
    has them (16-bit types, 64 or 128 output columns); by default such launches build
    the table on their first call, keep it with the metadata and use it unless the rows have at least 256 slots and every
    one of them starts on a multiple of 8 positions (blocked masks with large blocks: the general kernel is faster
    there); ``False`` always runs the general kernel.  The kernels agree up to the order of the float32 additions.
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
    arr = segs.seg_array(L, T)
    if plan is None and x.dtype in (torch.float16, torch.bfloat16) and output.dtype == x.dtype and n_out in (64, 128) \
            and (segs.has_plan(L, dev) or not torch.cuda.is_current_stream_capturing()) \
            and not (T >= 256 and segs.plan_is_aligned(L, dev)):  # (no table is built under stream capture: building synchronises)
        plan = segs.plan(L, dev)
    if plan is not None and plan is not False:
        _hip.require_device_tensor(plan, "plan")
        if plan.device != dev:
            raise _hip.SplatError(f"the plan lives on {plan.device}, the tensors on {dev}")
        with torch.cuda.device(dev):
            rc = _hip.lib().splat_spmm_planned(x.data_ptr(), y.data_ptr(), vs[0], vs[1], vs[2], output.data_ptr(), arr,
                                               len(segs), B, H, L, n_keys, n_out, T, _hip.dtype_code(x.dtype),
                                               _hip.dtype_code(output.dtype), plan.data_ptr(),
                                               plan.numel() * plan.element_size(), _hip.stream_ptr(dev))
        _hip.check(rc, "splat_spmm_planned")
        return (output, sTod_linear_transformations, sTod_translations, nnzs)
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_spmm(x.data_ptr(), y.data_ptr(), vs[0], vs[1], vs[2], output.data_ptr(), arr, len(segs),
                                   B, H, L, n_keys, n_out, T, _hip.dtype_code(x.dtype), _hip.dtype_code(output.dtype),
                                   _hip.stream_ptr(dev))
    _hip.check(rc, "splat_spmm")
    return (output, sTod_linear_transformations, sTod_translations, nnzs)


def is_correct(left_tensor: torch.Tensor, right_tensor: torch.Tensor, out_rspmm: torch.Tensor,
               sTod_linear_transofrmations: torch.Tensor, sTod_translations: torch.Tensor, nnzs: torch.Tensor,
               num_heads: int, batch_size: int, mask) -> bool:
    """``out_rspmm`` [B, H, L, n] against sum over the live slots s of left[.., r, s] * right[.., column of s, :], within
    1e-3 per entry.  The reference evaluates that sum with a Python loop per entry (its ``dot_product``) and only at the
    output columns whose index is a live mask column of the row; here every entry is checked, in float64 on the
    device.  Prints the reference's verdict lines and returns the verdict."""
    rows = len(mask) if not isinstance(mask, torch.Tensor) else mask.shape[0]
    dev = left_tensor.device
    T = left_tensor.shape[-1]
    n_keys = right_tensor.shape[2]
    first = getattr(sTod_translations, "splat_first_col", None)  # read before slicing: a slice drops the attribute
    cols, live = live_slot_columns(sTod_linear_transofrmations[:rows], sTod_translations[:rows], nnzs[:rows], T,
                                   None if first is None else first[:rows])
    cols, live = cols.clamp_(0, n_keys - 1).to(dev), live.to(dev)
    total, n_bad = 0.0, 0
    for b in range(batch_size):
        for h in range(num_heads):
            p = torch.where(live, left_tensor[b, h, :rows].double(), torch.zeros((), dtype=torch.float64, device=dev))
            dense = torch.zeros(rows, n_keys, dtype=torch.float64, device=dev).scatter_add_(1, cols, p)
            diff = (dense @ right_tensor[b, h].double() - out_rspmm[b, h, :rows].double().to(dev)).abs()
            bad = diff > 1e-3
            n_bad += int(bad.sum())
            total += float(diff[bad].sum())
    if n_bad > 0:
        print(f'test case failed average mse: {total}')
        return False
    print('test case passed!')
    return True


def test(m: int, k: int, n: int, num_heads: int, batch_size: int, mask, GPU_ID: Any, BLOCK_SIZE_Y: int,
         BLOCK_SIZE_X: int, output_dtype: torch.dtype) -> bool:
    """Compressed [m, T] times dense [k, n] per (batch, head) on integer-valued float32 inputs; returns ``is_correct``'s
    verdict (the reference drops it)."""
    assert m == n, "We only need to consider the case when m=n."
    (dTos_linear_transformations, dTos_translations, sTod_linear_transformations, sTod_translations, nnzs, _,
     span_loop_start, span_loop_end) = create_acsr(mask, BLOCK_SIZE_X, GPU_ID)
    output_tensor, grid_dim, trailing_dim_acsr = rspmm_preamble(mask, (batch_size, num_heads, m, n), BLOCK_SIZE_X,
                                                                BLOCK_SIZE_Y, GPU_ID, output_dtype)
    left = torch.randint(0, 100, (batch_size, num_heads, m, trailing_dim_acsr), dtype=torch.float32).to(GPU_ID)
    right = torch.randint(0, 100, (batch_size, num_heads, k, n), dtype=torch.float32).to(GPU_ID)
    rspmm_output, sTod_linear_transformations, sTod_translations, nnzs = rspmm_launcher(
        left, right, output_tensor, dTos_linear_transformations, dTos_translations, sTod_linear_transformations,
        sTod_translations, span_loop_start, span_loop_end, trailing_dim_acsr, nnzs, grid_dim, BLOCK_SIZE_Y, BLOCK_SIZE_X)
    return is_correct(left, right, rspmm_output, sTod_linear_transformations, sTod_translations, nnzs, num_heads,
                      batch_size, mask)
