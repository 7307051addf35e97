"""Regular (ACSR) sparse attention: SDDMM -> softmax -> SpMM, or the three fused into one kernel.

Mirrors the reference's ``SPLAT/r_attention.py``: ``RegularAttention`` (:12-100) keeps its constructor
signature, attribute names and ``forward([q, kT, v])``; ``unit`` (:102-110) keeps its signature.

Differences, all opt-in or invisible to a caller of the reference:
  * ``forward`` runs the fused online-softmax kernel by default (``fused=False`` gives the three launches);
    the two [B, H, L, T] intermediates are therefore allocated on first use, not in ``__init__``;
  * ``scale`` (default 1.0: the reference applies no softmax scale) multiplies the scores;
  * ``mask`` may be a list of lists (reference), an array / tensor, a ``MaskPattern`` or a list of
    ``MaskPattern`` segments (several affine segments per row).
"""
from __future__ import annotations

import contextlib
from typing import Any

import torch
import torch.nn as nn

import _splat_hip as _hip
from acsr_helpers import (ACSRSegments, MaskPattern, create_acsr, create_acsr_segments, create_blocked_mask,  # noqa: F401
                          create_causal_windowed_mask, create_windowed_mask, mask_shape, transpose_keys)
from r_sddmm import rsddmm_launcher, rsddmm_preamble
from r_softmax import rsoftmax_launcher, rsoftmax_preamble
from r_spmm import rspmm_launcher, rspmm_preamble


def _is_segment_list(mask) -> bool:
    return isinstance(mask, (list, tuple)) and len(mask) > 0 and isinstance(mask[0], (MaskPattern, torch.Tensor))


def attention_plan(segments: ACSRSegments, L: int, device) -> torch.Tensor:
    """The fused kernel's plan for these segments and ``L`` rows (which key tiles each 128-row block walks, every
    row's window): an opaque uint8 device tensor, built once per mask and handed to ``attention_launcher``."""
    return segments.plan(L, device)


_NO_GUARD = contextlib.nullcontext()


def attention_launcher(q: torch.Tensor, kT: torch.Tensor, v: torch.Tensor, output: torch.Tensor,
                       segments: ACSRSegments, scale: float = 1.0, plan: torch.Tensor | None = None,
                       lse: torch.Tensor | None = None) -> torch.Tensor:
    """Fused forward: output[b, h, r, :] = softmax over the live columns of (scale * q.kT)[b, h, r, :] times v.
    q [B, H, L, d], kT [B, H, d, L] (unit stride along d or along L), v [B, H, L, d], output [B, H, L, d];
    d in {64, 128}; one dtype for all four.  ``plan`` (from ``attention_plan`` for the same segments and L) spares
    every workgroup the derivation of its tiles from the ACSR arrays; the results are the same.  ``lse`` (float32
    [B, H, L], contiguous), when given, receives every row's log of the sum of exp(scale * score) over its live
    columns (+inf for a row without any), so that the row's probabilities are exp(scale * score - lse)."""
    for name, t in (("q", q), ("kT", kT), ("v", v), ("output", output)):
        _hip.require_device_tensor(t, name)
        if t.dim() != 4:
            raise _hip.SplatError(f"{name} must be 4-D")
    if not (q.dtype == kT.dtype == v.dtype == output.dtype):
        raise _hip.SplatError("q, kT, v and output must share a dtype")
    B, H, L, d = q.shape
    if tuple(kT.shape) != (B, H, d, L) or tuple(v.shape) != (B, H, L, d) or tuple(output.shape) != (B, H, L, d):
        raise _hip.SplatError(f"expected kT {(B, H, d, L)}, v and output {(B, H, L, d)}; got {tuple(kT.shape)}, "
                              f"{tuple(v.shape)}, {tuple(output.shape)}")
    if output.stride(3) != 1:
        raise _hip.SplatError("output needs unit stride along d")
    # The kernel moves 16-byte pieces: base addresses and batch / head / row strides must be multiples of 16 bytes.
    # Views that are not (odd storage offsets, row strides that are not a multiple of 8 or 4 elements) are copied.
    epc = 16 // q.element_size()

    def piecewise(t, strides):
        st = t.stride()
        return t.data_ptr() % 16 == 0 and all(st[i] % epc == 0 for i in strides)
    if q.stride(3) != 1 or not piecewise(q, (0, 1, 2)):
        q = q.contiguous()
    if v.stride(3) != 1 or not piecewise(v, (0, 1, 2)):
        v = v.contiguous()
    # Gathered rows: K row-major spares the walk over the keys in between (1.5 x at step 2, 8 x for config 3's far field;
    # the transposing copy costs a tenth of the kernel).
    kT = segments.keys_as_rows(kT)
    if kT.stride(2) == 1 and kT.stride(3) >= d and piecewise(kT, (0, 1, 3)):
        pass  # rows of K contiguous: [.., L, d] memory seen as [.., d, L]
    elif kT.stride(3) == 1 and L % epc == 0 and piecewise(kT, (0, 1, 2)):
        pass  # K^T contiguous along the keys, the reference's layout, in whole 16-byte pieces
    else:
        # e.g. the reference's contiguous [B, H, d, L] with L not a multiple of the piece: rows of K made contiguous
        kT = (transpose_keys(kT) if kT.stride(3) == 1 else kT.transpose(2, 3).contiguous()).transpose(2, 3)
    target = output
    if not piecewise(output, (0, 1, 2)):
        output = torch.empty((B, H, L, d), dtype=target.dtype, device=target.device)
    qs, ks, vs, os_ = q.stride(), kT.stride(), v.stride(), output.stride()
    dev = q.device
    arr = segments.seg_array(L)
    args = (q.data_ptr(), qs[0], qs[1], qs[2], kT.data_ptr(), ks[0], ks[1], ks[2], ks[3],
            v.data_ptr(), vs[0], vs[1], vs[2], output.data_ptr(), os_[0], os_[1], os_[2],
            arr, len(segments), B, H, L, d, float(scale), _hip.dtype_code(q.dtype))
    if plan is not None:
        _hip.require_device_tensor(plan, "plan")
        if plan.device != dev:
            raise _hip.SplatError(f"the plan lives on {plan.device}, the tensors on {dev}")
    if lse is not None:
        _hip.require_device_tensor(lse, "lse")
        if lse.dtype != torch.float32 or tuple(lse.shape) != (B, H, L) or not lse.is_contiguous() or lse.device != dev:
            raise _hip.SplatError(f"lse must be a contiguous float32 tensor of shape {(B, H, L)} on {dev}")
    # (the device guard costs 3-4 us of the call's 16 on the host: entered only when another device is current)
    with (_NO_GUARD if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)):
        if lse is not None:
            rc = _hip.lib().splat_attention_fwd_stats(*args, plan.data_ptr() if plan is not None else None,
                                                      plan.numel() * plan.element_size() if plan is not None else 0,
                                                      lse.data_ptr(), _hip.stream_ptr(dev))
            _hip.check(rc, "splat_attention_fwd_stats")
        elif plan is None:
            rc = _hip.lib().splat_attention_fwd(*args, _hip.stream_ptr(dev))
            _hip.check(rc, "splat_attention_fwd")
        else:
            rc = _hip.lib().splat_attention_fwd_planned(*args, plan.data_ptr(), plan.numel() * plan.element_size(),
                                                        _hip.stream_ptr(dev))
            _hip.check(rc, "splat_attention_fwd_planned")
    if target is not output:
        target.copy_(output)
    return target


class RegularAttention(nn.Module):

    def __init__(self, batch: int, seq_length: int, num_heads: int, head_dim: int, mask,
                 BLOCK_SIZE_Y: int, BLOCK_SIZE_X: int, GPU_ID: Any, out_dtype: torch.dtype,
                 *, scale: float | None = None, fused: bool = True):
        super().__init__()
        self._device = _hip.resolve_device(GPU_ID)
        self._mask = mask
        self._shape = (batch, num_heads, seq_length, head_dim)
        self._out_dtype = out_dtype
        self._GPU_ID = GPU_ID
        self.scale = 1.0 if scale is None else float(scale)
        self.fused = fused

        for m in (mask if _is_segment_list(mask) else [mask]):
            if tuple(mask_shape(m)) != (seq_length, seq_length):
                raise _hip.SplatError(f"the mask is {tuple(mask_shape(m))}, the module attends over "
                                      f"{(seq_length, seq_length)}: every kernel indexes the ACSR with the sequence's rows")
        if _is_segment_list(mask):
            self.segments = create_acsr_segments(mask, BLOCK_SIZE_Y, GPU_ID)
        else:
            t = create_acsr(mask, BLOCK_SIZE_Y, GPU_ID)
            self.segments = ACSRSegments([t], [t[3].splat_first_col])
        first = self.segments.tuples[0]

        # ACSR metadata of the (first) segment under the reference's attribute names.
        self.dTos_linear_transformations = first[0]
        self.dTos_translations = first[1]
        self.sTod_linear_transformations = first[2]
        self.sTod_translations = first[3]
        self.acsr_trailing_dim = self.segments.T
        self.nnzs = first[4]
        self.span_loop_start = first[6]
        self.span_loop_end = first[7]

        self.BLOCK_SIZE_Y = BLOCK_SIZE_Y
        self.BLOCK_SIZE_X = BLOCK_SIZE_X

        self.rspmm_output = torch.empty(self._shape, dtype=out_dtype, device=self._device)
        self.rspmm_grid_dim = (-(-head_dim // BLOCK_SIZE_X), -(-seq_length // BLOCK_SIZE_Y), batch * num_heads)
        self._unfused_ready = False
        self._plan = None  # the fused kernel's plan of this mask, built on the first fused forward
        self._segments_t = None  # ACSR of the transposed mask(s), built on the first backward
        self._plan_t = None  # the fused backward's plan of the transposed mask
        self._lse = None  # the rows' softmax statistics, allocated by the first forward_with_stats
        self._BLOCK_HEIGHT = BLOCK_SIZE_Y

    # The two [B, H, L, T] intermediates and the reference's launch geometry exist only for the unfused path.
    def _prepare_unfused(self):
        if self._unfused_ready:
            return
        B, H, L, _ = self._shape
        T = self.acsr_trailing_dim
        tile_mask = self._mask[0] if _is_segment_list(self._mask) else self._mask
        (self._rsddmm_output, self._rsddmm_grid_dim, self._rsddmm_tb_map_x,
         self._rsddmm_tb_map_y) = rsddmm_preamble(tile_mask, (B, H, L, T), self.BLOCK_SIZE_X, self.BLOCK_SIZE_Y,
                                                  self._GPU_ID, self._out_dtype)
        (self._rsoftmax_grid_dim, self._rsoftmax_output, _,
         self._rsoftmax_trailing_dim_pow_two) = rsoftmax_preamble(tile_mask, (B, H, L, T), self.BLOCK_SIZE_X,
                                                                  self._GPU_ID, self._out_dtype)
        self._unfused_ready = True

    def _lazy(name):  # noqa: N805
        def get(self):
            self._prepare_unfused()
            return getattr(self, "_" + name)
        return property(get)

    rsddmm_output = _lazy("rsddmm_output")
    rsddmm_grid_dim = _lazy("rsddmm_grid_dim")
    rsddmm_tb_map_x = _lazy("rsddmm_tb_map_x")
    rsddmm_tb_map_y = _lazy("rsddmm_tb_map_y")
    rsoftmax_output = _lazy("rsoftmax_output")
    rsoftmax_grid_dim = _lazy("rsoftmax_grid_dim")
    rsoftmax_trailing_dim_pow_two = _lazy("rsoftmax_trailing_dim_pow_two")
    del _lazy

    def forward(self, x):
        """x = [q, kT, v] after RoPE: q [B, H, L, d], kT [B, H, d, L], v [B, H, L, d].  Returns the module's
        output buffer (reused by every call)."""
        q, k, v = x
        fusable = self.fused and q.shape[-1] in (64, 128) and q.dtype == k.dtype == v.dtype == self._out_dtype
        if fusable:
            if self._plan is None:
                self._plan = attention_plan(self.segments, self._shape[2], self._device)
                # once, so that later forwards may run on any stream without ordering themselves after the plan kernel
                torch.cuda.current_stream(self._device).synchronize()
            return attention_launcher(q, k, v, self.rspmm_output, self.segments, self.scale, self._plan)

        multi = self.segments  # (also for one segment: the object keeps what every call would otherwise rebuild and recheck)
        rsddmm_launcher(q, k, self.rsddmm_output,
                        self.dTos_linear_transformations, self.dTos_translations,
                        self.sTod_linear_transformations, self.sTod_translations,
                        self.acsr_trailing_dim, self.nnzs,
                        self.rsddmm_grid_dim, self.rsddmm_tb_map_x,
                        self.rsddmm_tb_map_y, self.BLOCK_SIZE_Y, self.BLOCK_SIZE_X, scale=self.scale, segments=multi)
        rsoftmax_launcher(self.rsddmm_output, self.rsoftmax_output,
                          self.dTos_linear_transformations, self.dTos_translations,
                          self.sTod_linear_transformations, self.sTod_translations,
                          self.acsr_trailing_dim, self.rsoftmax_trailing_dim_pow_two, self.nnzs,
                          self.rsoftmax_grid_dim, self.BLOCK_SIZE_X, segments=multi)
        rspmm_launcher(self.rsoftmax_output, v, self.rspmm_output,
                       self.dTos_linear_transformations, self.dTos_translations,
                       self.sTod_linear_transformations, self.sTod_translations,
                       self.span_loop_start, self.span_loop_end, self.acsr_trailing_dim,
                       self.nnzs, self.rspmm_grid_dim, self.BLOCK_SIZE_Y, self.BLOCK_SIZE_X, segments=multi)
        return self.rspmm_output

    def forward_with_stats(self, x):
        """``forward(x)`` through the fused kernel plus every row's softmax statistic: returns ``(output, lse)`` with
        ``lse`` float32 [B, H, L] = log of the row's sum of exp(scale * score) over its live columns (+inf for a row
        without any).  Partial results over disjoint sets of keys merge exactly with it:
        ``out = sum_i exp(lse_i - logsumexp_i(lse_i)) * out_i``."""
        q, k, v = x
        if not (q.shape[-1] in (64, 128) and q.dtype == k.dtype == v.dtype == self._out_dtype):
            raise _hip.SplatError("the softmax statistic comes from the fused kernel: d in {64, 128}, one dtype")
        if self._plan is None:
            self._plan = attention_plan(self.segments, self._shape[2], self._device)
            torch.cuda.current_stream(self._device).synchronize()
        if self._lse is None:
            self._lse = torch.empty(self._shape[:3], dtype=torch.float32, device=self._device)
        attention_launcher(q, k, v, self.rspmm_output, self.segments, self.scale, self._plan, self._lse)
        return self.rspmm_output, self._lse

    def backward_pass(self, x, grad_out: torch.Tensor, lse: torch.Tensor | None = None, out: torch.Tensor | None = None,
                      fused: bool | None = None, sparse_rows: bool | None = None):
        """Gradients (dq, dk, dv), each [B, H, L, d], of ``forward(x)`` for x = [q, kT, v] and the upstream gradient
        ``grad_out`` [B, H, L, d].  The ACSR of the transposed mask is built on first use; see ``r_backward``.  ``lse``
        and ``out``: the rows' statistic and the output of ``forward_with_stats`` for the same x.  Where the fused
        forward applies (16-bit dtype, d in {64, 128}) the gradients come from the fused backward kernel, which needs both
        (a forward is run here when one is missing); otherwise, or with ``fused=False``, from the operators composed over
        compressed matrices, which ``lse`` spares the softmax pass.  ``sparse_rows``: how the fused kernel takes segments
        of the transposed mask that keep few keys with long columns (``r_backward.attention_backward_fused``)."""
        from r_backward import attention_backward, attention_backward_fused, transposed_segments
        q, kT, v = x
        if self._segments_t is None:
            masks = self._mask if _is_segment_list(self._mask) else [self._mask]
            self._segments_t = transposed_segments(masks, self._BLOCK_HEIGHT, self._GPU_ID)
        fusable = (self.fused and q.shape[-1] in (64, 128) and q.dtype in (torch.float16, torch.bfloat16) and
                   q.dtype == kT.dtype == v.dtype == grad_out.dtype == self._out_dtype)
        if fused is None:
            fused = fusable
        elif fused and not fusable:
            raise _hip.SplatError("the fused backward needs a 16-bit dtype shared by all tensors and d in {64, 128}")
        if not fused:
            return attention_backward(q, kT, v, grad_out, self.segments, self._segments_t, self.scale, lse)
        if lse is None or out is None:
            out, lse = self.forward_with_stats(x)
        if self._plan is None or self._plan_t is None:
            if self._plan is None:
                self._plan = attention_plan(self.segments, self._shape[2], self._device)
            if self._plan_t is None:
                self._plan_t = attention_plan(self._segments_t, self._shape[2], self._device)
            # once, so that later calls may run on any stream without ordering themselves after the plan kernels
            torch.cuda.current_stream(self._device).synchronize()
        return attention_backward_fused(q, kT, v, out, grad_out, lse, self.segments, self._segments_t, self._plan,
                                        self._plan_t, self.scale, sparse_rows)


class _AttentionFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, attn):
        ctx.attn = attn
        if attn.fused and q.shape[-1] in (64, 128) and q.dtype == k.dtype == v.dtype == attn._out_dtype:
            out, lse = attn.forward_with_stats([q, k.transpose(2, 3), v])
            out = out.clone()  # the module's buffers are reused by the next call
            ctx.save_for_backward(q, k, v, lse.clone(), out)
            return out
        out = attn([q, k.transpose(2, 3), v])
        ctx.save_for_backward(q, k, v)
        return out.clone()

    @staticmethod
    def backward(ctx, grad_out):
        q, k, v, *stat = ctx.saved_tensors
        dq, dk, dv = ctx.attn.backward_pass([q, k.transpose(2, 3), v], grad_out, stat[0] if stat else None,
                                            stat[1] if stat else None)
        return dq, dk, dv, None


def attention_with_grad(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, attn: RegularAttention) -> torch.Tensor:
    """``attn([q, k^T, v])`` for q, k, v [B, H, L, d] as a differentiable operation (fused forward, backward from
    ``RegularAttention.backward_pass``)."""
    return _AttentionFunction.apply(q, k, v, attn)


def unit(q, k, v, w_q, w_k, w_v, attn: RegularAttention):
    """Project [B, S, D] activations with [D, N, H] weights and attend.  The projections are laid out
    [B, N, S, H] (heads before sequence), which is the layout ``RegularAttention.forward`` documents;
    K is handed over as a transposed view, not a copy."""
    q = torch.einsum('bsd, dnh -> bnsh', q, w_q)
    k = torch.einsum('bsd, dnh -> bnsh', k, w_k)
    v = torch.einsum('bsd, dnh -> bnsh', v, w_v)
    return attn([q, k.transpose(2, 3), v])
