"""R-SDDMM: Q.K^T sampled onto the live slots of an ACSR.

Mirrors the reference's ``SPLAT/r_sddmm.py``: ``gen_block_mappings`` / ``naive_block_mappings`` (:117-151),
``rsddmm_preamble`` (:154-169) and ``rsddmm_launcher`` (:171-184) keep their names, positional parameters
and return tuples.  The Triton kernel (:15-115) is replaced by ``splat_sddmm`` (MFMA, gfx950).  The module's
self-check (``truth`` :186-188, ``is_correct`` :191-221, ``test`` :224-256) keeps its names, signatures and
acceptance rule; the four nested Python loops of the checker are tensor operations on the device here.
"""
from __future__ import annotations

from typing import Any

import numpy as np
import torch

import _splat_hip as _hip
from acsr_helpers import ACSRSegments, create_acsr, create_blocked_mask, mask_shape, row_extents  # noqa: F401


def naive_block_mappings(mask, BLOCK_HEIGHT: int, BLOCK_WIDTH: int, GPU_ID: Any) -> tuple[torch.Tensor, torch.Tensor]:
    """Anchor points (x = column, y = row) of the BLOCK_HEIGHT x BLOCK_WIDTH tiles that cover each row block's
    nonzero column range, as int32 device tensors -- the tiling the reference's launch grid is derived from.
    Its conventions are kept: max(rows // BLOCK_HEIGHT, 1) row blocks, anchors from the block's first
    nonzero column while strictly below its last one."""
    dev = _hip.resolve_device(GPU_ID)
    rows, cols = mask_shape(mask)
    first, last = row_extents(mask, dev)
    first, last = first.cpu().numpy().astype(np.int64), last.cpu().numpy().astype(np.int64)
    n_blocks = max(rows // BLOCK_HEIGHT, 1)
    pad = n_blocks * BLOCK_HEIGHT - min(rows, n_blocks * BLOCK_HEIGHT)
    f = np.concatenate([first[:n_blocks * BLOCK_HEIGHT], np.full(pad, cols)]).reshape(n_blocks, BLOCK_HEIGHT)
    l = np.concatenate([last[:n_blocks * BLOCK_HEIGHT], np.full(pad, -1)]).reshape(n_blocks, BLOCK_HEIGHT)
    lo = np.minimum(f.min(axis=1), cols)
    hi = np.maximum(l.max(axis=1), 0)
    counts = np.where(hi > lo, -(-(hi - lo) // BLOCK_WIDTH), 0)
    total = int(counts.sum())
    assert total > 0, "Issues with generating arrangement!"
    blk = np.repeat(np.arange(n_blocks), counts)
    within = np.arange(total) - np.repeat(np.cumsum(counts) - counts, counts)
    xs = (lo[blk] + within * BLOCK_WIDTH).astype(np.int32)
    ys = (blk * BLOCK_HEIGHT).astype(np.int32)
    return torch.from_numpy(xs).to(dev), torch.from_numpy(ys).to(dev)


def gen_block_mappings(mask, BLOCK_HEIGHT: int, BLOCK_WIDTH: int, GPU_ID: Any,
                       is_naive: bool = True) -> tuple[torch.Tensor, torch.Tensor]:
    return naive_block_mappings(mask, BLOCK_HEIGHT, BLOCK_WIDTH, GPU_ID)


def rsddmm_preamble(mask, output_shape: tuple[int], BLOCK_SIZE_X: int, BLOCK_SIZE_Y: int, GPU_ID: Any,
                    out_dtype: torch.dtype):
    """-> (output [B, H, L, T] uninitialised, grid_dim = (n_tiles, B*H), tb_map_x, tb_map_y)."""
    dev = _hip.resolve_device(GPU_ID)
    output = torch.empty(tuple(output_shape), dtype=out_dtype, device=dev)
    tb_map_x, tb_map_y = gen_block_mappings(mask, BLOCK_SIZE_Y, BLOCK_SIZE_X, GPU_ID)
    assert tb_map_x.shape == tb_map_y.shape, "Incorrect tiling arrangement!"
    grid_dim = (tb_map_x.shape[0], output_shape[0] * output_shape[1])
    return (output, grid_dim, tb_map_x, tb_map_y)


def _strides4(t: torch.Tensor, name: str):
    if t.dim() != 4:
        raise _hip.SplatError(f"{name} must be 4-D [batch, heads, ., .]")
    return t.stride()


def _takes_a_plan(x, output, y, B: int, H: int, L: int, d: int, T: int, segs: ACSRSegments) -> bool:
    """Whether this launch runs the kernel that reads a plan table (the library decides by the same rules and ignores the
    plan otherwise): 16-bit types, d = 64 / 128, rows of K contiguous, 16-byte alignment, and at least 256 row blocks or rows
    of at most 256 slots (fewer blocks of longer rows are better off with the general kernel's split of the key range)."""
    if x.dtype not in (torch.float16, torch.bfloat16) or output.dtype != x.dtype or d not in (64, 128):
        return False
    if y.stride(2) != 1 or T % 8 != 0 or any(off % 8 for off in segs.offsets):
        return False
    return B * H * ((L + 127) // 128) >= 256 or T <= 256


def rsddmm_launcher(x: torch.Tensor, y: torch.Tensor, output: torch.Tensor,
                    dTos_linear_transformations: torch.Tensor, dTos_translations: torch.Tensor,
                    sTod_linear_transformations: torch.Tensor, sTod_translations: torch.Tensor,
                    trailing_dim: int, nnzs: torch.Tensor, grid_dim: tuple[int],
                    tb_map_x: torch.Tensor, tb_map_y: torch.Tensor,
                    BLOCK_SIZE_Y: int, BLOCK_SIZE_X: int, *, scale: float | None = None,
                    segments: ACSRSegments | None = None, lse: torch.Tensor | None = None,
                    plan: torch.Tensor | None | bool = None):
    """x = Q [B, H, L, d]; y = K^T [B, H, d, L] (any strides with unit stride along d or along L, so
    ``k.transpose(2, 3)`` of a [B, H, L, d] tensor needs no copy); output [B, H, L, T] is written in place for
    the live slots only.  ``grid_dim`` / ``tb_map_*`` / ``BLOCK_SIZE_*`` describe the reference's launch
    geometry and are accepted unchanged; the HIP kernel tiles by itself from the row maps.  With ``lse`` (float32
    [B, H, L], contiguous: every row's log of its sum of exp(scale * score), as the fused forward hands it out) the
    stored value is exp(scale * score - lse[row]), the row's softmax probability, instead of the score.
    ``plan``: the mask's plan table (``ACSRSegments.plan``); by default the launches that use one (16-bit types, d = 64 or
    128, at least 256 row blocks of 128 rows or rows of at most 256 slots) build it on their first call and keep it with the metadata, ``False``
    launches without one.  The results are the same bit for bit.
    Returns (output, sTod_linear_transformations, sTod_translations, nnzs)."""
    for name, t in (("x", x), ("y", y), ("output", output)):
        _hip.require_device_tensor(t, name)
    if x.dtype != y.dtype:
        raise _hip.SplatError("x and y must share a dtype")
    segs = segments or ACSRSegments.single(dTos_linear_transformations, dTos_translations,
                                           sTod_linear_transformations, sTod_translations, nnzs, trailing_dim)
    B, H, L, d = x.shape
    if y.shape[0] != B or y.shape[1] != H or y.shape[2] != d:
        raise _hip.SplatError(f"y must be [B, H, d, n] = [{B}, {H}, {d}, n], got {tuple(y.shape)}")
    n_keys = y.shape[3]
    if x.stride(3) != 1 and d > 1:
        x = x.contiguous()
    if y.stride(2) != 1 and y.stride(3) != 1:
        y = y.contiguous()
    y = segs.keys_as_rows(y)  # gathered rows: K row-major spares the walk over the keys in between (3 x at step 2)
    if not output.is_contiguous() or tuple(output.shape) != (B, H, L, trailing_dim):
        raise _hip.SplatError(f"output must be a contiguous [B, H, L, T] = {(B, H, L, trailing_dim)} tensor")
    qs, ks = _strides4(x, "x"), _strides4(y, "y")
    dev = x.device
    arr = segs.seg_array(L, trailing_dim)
    args = (x.data_ptr(), qs[0], qs[1], qs[2], y.data_ptr(), ks[0], ks[1], ks[2], ks[3], output.data_ptr(), arr, len(segs),
            B, H, L, n_keys, d, trailing_dim, 1.0 if scale is None else float(scale), _hip.dtype_code(x.dtype),
            _hip.dtype_code(output.dtype))
    if lse is not None:
        _hip.require_device_tensor(lse, "lse")
        if lse.dtype != torch.float32 or tuple(lse.shape) != (B, H, L) or not lse.is_contiguous() or lse.device != dev:
            raise _hip.SplatError(f"lse must be a contiguous float32 tensor of shape {(B, H, L)} on {dev}")
    # (building the table synchronises once, which a stream under capture must not do: such a call uses a table only if an
    # earlier call has left one)
    if plan is None and _takes_a_plan(x, output, y, B, H, L, d, trailing_dim, segs) \
            and (segs.has_plan(L, dev) or not torch.cuda.is_current_stream_capturing()):
        plan = segs.plan(L, dev)
    if plan is not None and plan is not False:
        _hip.require_device_tensor(plan, "plan")
        if plan.device != dev:
            raise _hip.SplatError(f"the plan lives on {plan.device}, the tensors on {dev}")
        with torch.cuda.device(dev):
            rc = _hip.lib().splat_sddmm_planned(*args, lse.data_ptr() if lse is not None else None, plan.data_ptr(),
                                                plan.numel() * plan.element_size(), _hip.stream_ptr(dev))
            _hip.check(rc, "splat_sddmm_planned")
        return (output, sTod_linear_transformations, sTod_translations, nnzs)
    with torch.cuda.device(dev):
        if lse is None:
            rc = _hip.lib().splat_sddmm(*args, _hip.stream_ptr(dev))
            _hip.check(rc, "splat_sddmm")
        else:
            rc = _hip.lib().splat_sddmm_probs(*args, lse.data_ptr(), _hip.stream_ptr(dev))
            _hip.check(rc, "splat_sddmm_probs")
    return (output, sTod_linear_transformations, sTod_translations, nnzs)


def live_slot_columns(sTod_linear_transformations: torch.Tensor, sTod_translations: torch.Tensor, nnzs: torch.Tensor,
                      trailing_dim: int, first_col: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """(columns int64 [rows, T], live bool [rows, T]): the dense column behind every compressed slot by the builder's
    rule c = sTod_lin * (s + sTod_trans) (acsr_helpers.py:122-124; for unit steps the same as the reference checkers'
    round(s * lin + trans), r_sddmm.py:210), and which slots are live (s < nnz).  Rows with one live column store
    translation 0 whatever the column is; their column is taken from ``first_col`` (int tensor [rows]) or, when that is
    not given, from the builder's ``splat_first_col`` attribute of ``sTod_translations`` (a slice or copy of that tensor
    no longer carries the attribute, so callers that slice pass ``first_col`` themselves)."""
    lin = sTod_linear_transformations.double()
    trans = sTod_translations.double()
    slots = torch.arange(trailing_dim, device=lin.device, dtype=torch.float64)
    cols = torch.round(lin[:, None] * (slots[None, :] + trans[:, None])).long()
    live = slots[None, :] < nnzs.double()[:, None]
    first = first_col if first_col is not None else getattr(sTod_translations, "splat_first_col", None)
    if first is not None:
        single = nnzs == 1
        cols[single, 0] = first.to(cols.device).long()[single]
    return cols, live


def truth(x: torch.Tensor, y: torch.Tensor, GPU_ID: Any) -> torch.Tensor:
    """The dense product the sampled one is checked against."""
    return torch.einsum('bnqd, bndk -> bnqk', x, y)


def is_correct(out_torch: torch.Tensor, out_rsddmm: torch.Tensor,
               sTod_linear_transofrmations: torch.Tensor, sTod_translations: torch.Tensor, nnzs: torch.Tensor,
               batch_size: int, num_heads: int, mask) -> bool:
    """Every live slot of ``out_rsddmm`` [B, H, L, T] must lie within 1e-3 of the dense product's entry at the slot's
    column.  Prints the reference's verdict lines and returns the verdict."""
    rows = len(mask) if not isinstance(mask, torch.Tensor) else mask.shape[0]
    T = out_rsddmm.shape[-1]
    first = getattr(sTod_translations, "splat_first_col", None)  # read before slicing: a slice drops the attribute
    cols, live = live_slot_columns(sTod_linear_transofrmations[:rows], sTod_translations[:rows], nnzs[:rows], T,
                                   None if first is None else first[:rows])
    cols = cols.clamp_(0, out_torch.shape[-1] - 1).to(out_torch.device)
    want = out_torch[:batch_size, :num_heads, :rows].double().gather(3, cols.expand(batch_size, num_heads, rows, T))
    diff = (want - out_rsddmm[:batch_size, :num_heads, :rows].double().to(want.device)).abs()
    bad = (diff > 1e-3) & live.to(diff.device)
    if bool(bad.any()):
        print(f'test case failed average mse: {float(diff[bad].sum())}')
        return False
    print('test case passed!')
    return True


def test(m: int, k: int, n: int, num_heads: int, batch_size: int, mask, GPU_ID: Any, BLOCK_SIZE_Y: int,
         BLOCK_SIZE_X: int, out_dtype: torch.dtype) -> bool:
    """[m, k] x [k, n] per (batch, head) on integer-valued inputs, sampled onto ``mask``; returns ``is_correct``'s verdict
    (the reference drops it)."""
    assert m == n, "We only need to consider the case when m=n."
    left = torch.randint(0, 100, (batch_size, num_heads, m, k), dtype=out_dtype).to(GPU_ID)
    right = torch.randint(0, 100, (batch_size, num_heads, k, n), dtype=out_dtype).to(GPU_ID)
    (dTos_linear_transformations, dTos_translations, sTod_linear_transformations, sTod_translations, nnzs,
     acsr_trailing_dimension, _, _) = create_acsr(mask, BLOCK_SIZE_X, GPU_ID)
    output_tensor, grid_dim, tb_map_x, tb_map_y = rsddmm_preamble(mask, (batch_size, num_heads, m, acsr_trailing_dimension),
                                                                  BLOCK_SIZE_X, BLOCK_SIZE_Y, GPU_ID, out_dtype)
    rsddmm_output, sTod_linear_transformations, sTod_translations, nnzs = rsddmm_launcher(
        left, right, output_tensor, dTos_linear_transformations, dTos_translations, sTod_linear_transformations,
        sTod_translations, acsr_trailing_dimension, nnzs, grid_dim, tb_map_x, tb_map_y, BLOCK_SIZE_Y, BLOCK_SIZE_X)
    torch_output = truth(left, right, GPU_ID)
    return is_correct(torch_output, rsddmm_output, sTod_linear_transformations, sTod_translations, nnzs, batch_size,
                      num_heads, mask)
