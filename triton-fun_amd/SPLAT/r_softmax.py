"""R-Softmax: row softmax over the live slots of compressed score rows.

Mirrors the reference's ``SPLAT/r_softmax.py``: ``rsoftmax_preamble`` (:108-124, note the grid comes
first in its return tuple) and ``rsoftmax_launcher`` (:126-150).  The Triton kernels (:16-106) are
replaced by ``splat_softmax`` (one wavefront per row, every row is processed).  The module's self-check
(``is_correct`` :152-185, ``test`` :188-224) keeps its names, signatures and acceptance rule.
"""
from __future__ import annotations

from math import ceil, log2
from typing import Any

import torch

import _splat_hip as _hip
from acsr_helpers import ACSRSegments, create_acsr, create_blocked_mask, create_windowed_mask, mask_shape  # noqa: F401


def rsoftmax_preamble(mask, output_shape: tuple[int], BLOCK_SIZE_X: int, GPU_ID: Any, out_dtype: torch.dtype):
    """-> (grid_dim = (ceil(rows / BLOCK_SIZE_X), B*H), output [B, H, L, T] uninitialised, full_shape,
    T rounded up to a power of two)."""
    dev = _hip.resolve_device(GPU_ID)
    trailing_dim_pow_two = 2 ** ceil(log2(output_shape[-1]))
    full_shape = output_shape
    output = torch.empty(tuple(full_shape), dtype=out_dtype, device=dev)
    rows = mask_shape(mask)[0]
    grid_dim = (-(-rows // BLOCK_SIZE_X), output_shape[0] * output_shape[1])
    return (grid_dim, output, full_shape, trailing_dim_pow_two)


def rsoftmax_launcher(x: torch.Tensor, output: torch.Tensor,
                      dTos_linear_transformations: torch.Tensor, dTos_translations: torch.Tensor,
                      sTod_linear_transformations: torch.Tensor, sTod_translations: torch.Tensor,
                      acsr_trailing_dim_true: int, acsr_trailing_dim_power_two: int,
                      nnzs: torch.Tensor, grid_dim: tuple[int], BLOCK_SIZE_X: int, *,
                      segments: ACSRSegments | None = None):
    """x, output: [B, H, L, T] (output may be x).  Live slots of every row are normalised; dead slots are
    neither read nor written.  Returns (output, sTod_linear_transformations, sTod_translations, nnzs)."""
    _hip.require_device_tensor(x, "x")
    _hip.require_device_tensor(output, "output")
    if x.dim() != 4 or tuple(x.shape) != tuple(output.shape) or x.shape[3] != acsr_trailing_dim_true:
        raise _hip.SplatError(f"x and output must both be [B, H, L, T={acsr_trailing_dim_true}], got {tuple(x.shape)} "
                              f"and {tuple(output.shape)}")
    if not output.is_contiguous():
        raise _hip.SplatError("output must be contiguous")
    if not x.is_contiguous():
        x = x.contiguous()
    segs = segments or ACSRSegments.single(dTos_linear_transformations, dTos_translations,
                                           sTod_linear_transformations, sTod_translations, nnzs,
                                           acsr_trailing_dim_true)
    B, H, L, T = x.shape
    dev = x.device
    arr = segs.seg_array(L, T)
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_softmax(x.data_ptr(), output.data_ptr(), arr, len(segs), B * H, L, T,
                                      _hip.dtype_code(x.dtype), _hip.dtype_code(output.dtype), _hip.stream_ptr(dev))
    _hip.check(rc, "splat_softmax")
    return (output, sTod_linear_transformations, sTod_translations, nnzs)


def is_correct(inp_tensor: torch.Tensor, out_rsoftmax: torch.Tensor, sTod_linear_transofrmations: torch.Tensor,
               sTod_translations: torch.Tensor, nnzs: torch.Tensor, batch_size: int, num_heads: int, mask) -> bool:
    """The live slots of every row of ``out_rsoftmax`` [B, H, L, T] must sum to 1 within 1e-2 (the reference's rule: it
    checks the sums, not the values).  Prints the reference's verdict lines and returns the verdict."""
    rows = len(mask) if not isinstance(mask, torch.Tensor) else mask.shape[0]
    out = out_rsoftmax[:batch_size, :num_heads, :rows].double()
    T = out.shape[-1]
    live = torch.arange(T, device=out.device)[None, :] < nnzs[:rows].to(out.device)[:, None]
    sums = torch.where(live, out, torch.zeros((), dtype=out.dtype, device=out.device)).sum(-1)
    off = (sums - 1).abs()
    bad = off >= 1e-2
    if bool(bad.any()):
        print(f'test case failed average mse: {float(off[bad].sum())}')
        return False
    print('test case passed!')
    return True


def test(m: int, n: int, num_heads: int, batch_size: int, mask, GPU_ID: Any, BLOCK_SIZE_X: int,
         out_dtype: torch.dtype) -> bool:
    """Softmax over the compressed rows of an [m, n] mask on integer-valued float32 inputs; returns ``is_correct``'s
    verdict (the reference drops it)."""
    assert m == n, "We only need to consider the case when m=n."
    (dTos_linear_transformations, dTos_translations, sTod_linear_transformations, sTod_translations, nnzs,
     trailing_dim_acsr, _, _) = create_acsr(mask, BLOCK_SIZE_X, GPU_ID)
    grid_dim, output, full_shape, trailing_dim_pow_two = rsoftmax_preamble(
        mask, (batch_size, num_heads, m, trailing_dim_acsr), BLOCK_SIZE_X, GPU_ID, out_dtype)
    inp = torch.randint(0, 100, full_shape, dtype=torch.float32).to(GPU_ID)
    rsoftmax_output, sTod_linear_transformations, sTod_translations, nnzs = rsoftmax_launcher(
        inp, output, dTos_linear_transformations, dTos_translations, sTod_linear_transformations, sTod_translations,
        trailing_dim_acsr, trailing_dim_pow_two, nnzs, grid_dim, BLOCK_SIZE_X)
    return is_correct(inp, rsoftmax_output, sTod_linear_transformations, sTod_translations, nnzs, batch_size, num_heads,
                      mask)
