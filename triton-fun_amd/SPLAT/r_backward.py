"""Backward pass of ACSR sparse attention, composed from the forward operators plus two kernels of its own.

The reference stops at the forward (``r_attention.py:77-100``); this module gives the gradients of
``out = softmax_over_live_columns(scale * q.kT) . v`` with respect to q, k and v.  Everything stays in the compressed
[B, H, L, T] layout:

    S~  = rsddmm(q, kT) * scale            P~ = rsoftmax(S~)      (or P~ = exp(S~ - lse) in one pass, given the forward's lse)
    dP~ = rsddmm(dO, v^T)                  dS~ = P~ o (dP~ - rowsum(P~ o dP~)) * scale     (splat_softmax_bwd)
    dQ  = rspmm(dS~, k)
    dV  = P~^T . dO                        dK = dS~^T . q                                   (splat_spmm_t)

The transposed products read the compressed matrices as they are and take the ACSR of the transposed mask to know
which rows a column meets (``compressed_transpose_launcher`` can also store a matrix in that ACSR's layout, after which
``rspmm_launcher`` gives the same products).  The transposed mask must have affine rows as well, which holds for every
closed-form pattern (band, blocked, dilated, strided); for arbitrary affine-row masks it need not, and the gradients
with respect to k and v would then be wrong: ``transposed_segments`` checks every row of a transposed mask that came as
an array or tensor against its metadata and raises ``SplatError`` instead.
"""
from __future__ import annotations

from typing import Any, Sequence

import numpy as np
import torch

import _splat_hip as _hip
from acsr_helpers import ACSRSegments, MaskPattern, build_acsr, create_acsr_segments, non_affine_rows, transpose_keys
from r_sddmm import rsddmm_launcher
from r_softmax import rsoftmax_launcher
from r_spmm import rspmm_launcher


def transposed_mask(mask, device: Any):
    """mask^T: the transposed pattern for a closed-form pattern (nothing is rasterised), else a contiguous uint8 device
    tensor."""
    dev = _hip.resolve_device(device)
    if isinstance(mask, MaskPattern):
        return mask.transposed()
    if isinstance(mask, torch.Tensor):
        m = mask.to(device=dev, dtype=torch.uint8)
    else:
        m = torch.from_numpy(np.ascontiguousarray(np.asarray(mask), dtype=np.uint8)).to(dev)
    return m.t().contiguous()


def transposed_segments(masks: Sequence, BLOCK_HEIGHT: int, GPU_ID: Any) -> ACSRSegments:
    """The ACSR of the transpose of every segment mask, in the same order.  A mask whose transpose has a row that is not
    an arithmetic progression of columns (the mask's rows may all be affine while its columns are not) cannot be walked
    from that ACSR: ``SplatError``.  Closed-form patterns are exempt: their transposes are closed-form too."""
    dev = _hip.resolve_device(GPU_ID)
    t_masks = [transposed_mask(m, GPU_ID) for m in masks]
    for k, tm in enumerate(t_masks):
        if isinstance(tm, MaskPattern):
            continue
        b = build_acsr(tm, BLOCK_HEIGHT, dev)
        bad = non_affine_rows(tm, b.row_first, b.sTod_lin, b.nnz)
        if bad.numel() > 0:
            raise _hip.SplatError(
                f"segment {k}: {bad.numel()} column(s) of the mask (the first is column {int(bad[0])}) meet rows that do not "
                "form an arithmetic progression, so the transposed mask has no ACSR and the gradients with respect to k "
                "and v cannot be computed from it; split the mask into segments whose columns are affine as well")
    return create_acsr_segments(t_masks, BLOCK_HEIGHT, GPU_ID)


def softmax_backward_launcher(p: torch.Tensor, dp: torch.Tensor, ds: torch.Tensor, segments: ACSRSegments,
                              scale: float = 1.0) -> torch.Tensor:
    """ds[.., r, s] = p * (dp - sum over the row's live slots of p * dp) * scale; [B, H, L, T] contiguous tensors of
    one dtype; ``ds`` may be ``dp``."""
    for name, t in (("p", p), ("dp", dp), ("ds", ds)):
        _hip.require_device_tensor(t, name)
        if t.dim() != 4 or not t.is_contiguous() or tuple(t.shape) != tuple(p.shape) or t.dtype != p.dtype:
            raise _hip.SplatError(f"{name} must be a contiguous [B, H, L, T] tensor like p")
    B, H, L, T = p.shape
    if T != segments.T:
        raise _hip.SplatError(f"trailing dimension {T} does not match the segments' {segments.T}")
    dev = p.device
    arr = segments.seg_array(L, T)
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_softmax_bwd(p.data_ptr(), dp.data_ptr(), ds.data_ptr(), arr, len(segments), B * H, L, T,
                                          float(scale), _hip.dtype_code(p.dtype), _hip.stream_ptr(dev))
    _hip.check(rc, "splat_softmax_bwd")
    return ds


def compressed_transpose_launcher(src: torch.Tensor, dst: torch.Tensor, segments: ACSRSegments,
                                  segments_t: ACSRSegments) -> torch.Tensor:
    """src [B, H, L, T] in the layout of ``segments`` -> dst [B, H, Lt, Tt] in the layout of ``segments_t`` (the ACSR
    of the transposed segment masks): dst[j, t] is the entry of src that sits at (row i(j, t), column j)."""
    for name, t in (("src", src), ("dst", dst)):
        _hip.require_device_tensor(t, name)
        if t.dim() != 4 or not t.is_contiguous():
            raise _hip.SplatError(f"{name} must be a contiguous 4-D tensor")
    if src.dtype != dst.dtype or src.shape[:2] != dst.shape[:2] or len(segments) != len(segments_t):
        raise _hip.SplatError("src and dst must share dtype, batch and heads; both ACSRs the same number of segments")
    B, H, L, T = src.shape
    Lt, Tt = dst.shape[2], dst.shape[3]
    if T != segments.T or Tt != segments_t.T:
        raise _hip.SplatError("trailing dimensions do not match the segments")
    dev = src.device
    a, b = segments.seg_array(L, T), segments_t.seg_array(Lt, Tt)
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_compressed_transpose(src.data_ptr(), dst.data_ptr(), a, b, len(segments), B * H, L, T, Lt, Tt,
                                                   _hip.dtype_code(src.dtype), _hip.stream_ptr(dev))
    _hip.check(rc, "splat_compressed_transpose")
    return dst


def _rows_step_like_the_blocks(segments: ACSRSegments, segments_t: ACSRSegments) -> bool:
    """Whether the kernel of thin wavefronts is the faster one for these masks: it reads a row's entries at a block of
    output rows as consecutive slots when the row's column step equals the stride by which the transposed mask's rows are
    grouped into blocks (1 for windows and blocks, the dilation for dilated windows); rows of another step (the far field
    of a strided pattern) it walks a second time, entry by entry, which the general kernel does better."""
    strides = {int(getattr(t[3], "splat_row_stride", 1)) for t in segments_t.tuples}
    rs = strides.pop() if len(strides) == 1 else 1
    return segments.max_step <= 1 or segments.max_step == rs


def rspmm_t_launcher(p: torch.Tensor, x: torch.Tensor, out: torch.Tensor, segments: ACSRSegments,
                     segments_t: ACSRSegments, plan: torch.Tensor | None | bool = None) -> torch.Tensor:
    """out[.., j, :] = sum over the rows i that keep column j of p[.., i, slot of j in row i] * x[.., i, :], i.e. the
    product with the transposed compressed matrix: p [B, H, L, T] contiguous in the layout of ``segments``, x
    [B, H, L, n] with unit stride along n, out [B, H, Lt, n] contiguous; ``segments_t`` the ACSR of the transposed
    segment masks.  ``plan``: the plan table of the transposed mask (``segments_t.plan(Lt, device)``), which selects the
    kernel of thin wavefronts where the library has one (16-bit types, n = 64 / 128); None builds it on the first such call and keeps it with the metadata, False runs without."""
    for name, t in (("p", p), ("x", x), ("out", out)):
        _hip.require_device_tensor(t, name)
        if t.dim() != 4:
            raise _hip.SplatError(f"{name} must be a 4-D tensor")
    if not p.is_contiguous() or not out.is_contiguous():
        raise _hip.SplatError("p and out must be contiguous")
    if x.stride(3) != 1:
        raise _hip.SplatError("x needs unit stride along its last dimension")
    B, H, L, T = p.shape
    Lt, n = out.shape[2], out.shape[3]
    if tuple(x.shape) != (B, H, L, n) or tuple(out.shape[:2]) != (B, H) or x.dtype != p.dtype:
        raise _hip.SplatError(f"shapes do not fit: p {tuple(p.shape)}, x {tuple(x.shape)}, out {tuple(out.shape)}")
    if T != segments.T or len(segments) != len(segments_t):
        raise _hip.SplatError("the segments do not fit p (trailing dimension, number of segments)")
    dev = p.device
    a, b = segments.seg_array(L, T), segments_t.seg_array(Lt)
    xs = x.stride()
    if plan is None and p.dtype in (torch.float16, torch.bfloat16) and out.dtype == p.dtype and n in (64, 128) \
            and _rows_step_like_the_blocks(segments, segments_t) \
            and (segments_t.has_plan(Lt, dev) or not torch.cuda.is_current_stream_capturing()):
        plan = segments_t.plan(Lt, dev)  # (no table is built under stream capture: building synchronises)
    with torch.cuda.device(dev):
        if plan is not None and plan is not False:
            _hip.require_device_tensor(plan, "plan")
            if plan.device != dev:
                raise _hip.SplatError(f"the plan lives on {plan.device}, the tensors on {dev}")
            rc = _hip.lib().splat_spmm_t_planned(p.data_ptr(), x.data_ptr(), xs[0], xs[1], xs[2], out.data_ptr(), a, b,
                                                 len(segments), B, H, L, Lt, n, T, _hip.dtype_code(p.dtype),
                                                 _hip.dtype_code(out.dtype), plan.data_ptr(),
                                                 plan.numel() * plan.element_size(), _hip.stream_ptr(dev))
            _hip.check(rc, "splat_spmm_t_planned")
        else:
            rc = _hip.lib().splat_spmm_t(p.data_ptr(), x.data_ptr(), xs[0], xs[1], xs[2], out.data_ptr(), a, b, len(segments),
                                         B, H, L, Lt, n, T, _hip.dtype_code(p.dtype), _hip.dtype_code(out.dtype),
                                         _hip.stream_ptr(dev))
            _hip.check(rc, "splat_spmm_t")
    return out


def _sddmm(x, y, out, segs, scale, lse=None):
    rsddmm_launcher(x, y, out, None, None, None, None, segs.T, None, None, None, None, 16, 16, scale=scale, segments=segs,
                    lse=lse)


def _spmm(p, v, out, segs):
    rspmm_launcher(p, v, out, None, None, None, None, None, None, segs.T, None, None, 16, 16, segments=segs)


def attention_backward(q: torch.Tensor, kT: torch.Tensor, v: torch.Tensor, grad_out: torch.Tensor,
                       segments: ACSRSegments, segments_t: ACSRSegments, scale: float = 1.0,
                       lse: torch.Tensor | None = None):
    """(dq, dk, dv), each [B, H, L, d], for out = softmax_over_live_columns(scale * q.kT) . v and the upstream gradient
    ``grad_out`` [B, H, L, d].  q, v [B, H, L, d]; kT [B, H, d, L] (a view or a copy); one dtype throughout.  The
    probabilities are recomputed, as the fused forward never materialises them: by SDDMM + softmax, or, with the rows'
    statistic ``lse`` [B, H, L] of the forward (``RegularAttention.forward_with_stats``), by one SDDMM that stores
    exp(scale * score - lse)."""
    B, H, L, d = q.shape
    dt, dev = q.dtype, q.device
    k = kT.transpose(2, 3)
    if k.stride(3) != 1:
        k = k.contiguous()
    grad_out = grad_out.contiguous() if grad_out.stride(3) != 1 else grad_out
    T = segments.T
    probs = torch.empty((B, H, L, T), dtype=dt, device=dev)
    _sddmm(q, kT, probs, segments, scale, lse)
    if lse is None:
        rsoftmax_launcher(probs, probs, None, None, None, None, T, 0, None, None, 16, segments=segments)
    dprobs = torch.empty_like(probs)
    _sddmm(grad_out, v.transpose(2, 3), dprobs, segments, 1.0)
    softmax_backward_launcher(probs, dprobs, dprobs, segments, scale)  # dprobs now holds dS~
    dq = torch.empty((B, H, L, d), dtype=dt, device=dev)
    _spmm(dprobs, k, dq, segments)
    dv = torch.empty((B, H, L, d), dtype=dt, device=dev)
    rspmm_t_launcher(probs, grad_out, dv, segments, segments_t)
    dk = torch.empty((B, H, L, d), dtype=dt, device=dev)
    rspmm_t_launcher(dprobs, q if q.stride(3) == 1 else q.contiguous(), dk, segments, segments_t)
    return dq, dk, dv


class KeysSideSchedule:
    """How the fused backward walks a transposed mask some of whose segments keep only a few keys (rows), each with a long
    column of queries: ``main`` holds the other segments (walked by 128 consecutive keys as usual), and the live rows of the
    sparse segments are listed one per (key, stretch of queries): ``rows`` is their single-segment ACSR (``n_rows`` rows;
    stretch c owns rows [c * per_stretch, (c + 1) * per_stretch), the keys in the same order in every stretch),
    ``key_of_row`` the key each row belongs to (int32, -1 for padding rows, which are empty) and ``keys`` the
    listed keys (int64, distinct, ``len(keys) <= per_stretch``)."""

    def __init__(self, main: ACSRSegments, rows: ACSRSegments, key_of_row: torch.Tensor, keys: torch.Tensor,
                 n_stretches: int, per_stretch: int):
        self.main, self.rows, self.key_of_row, self.keys = main, rows, key_of_row, keys
        self.n_stretches, self.per_stretch = n_stretches, per_stretch
        self.n_rows = n_stretches * per_stretch


# a segment of the transposed mask is listed row by row when at most one row in this many is live
_SPARSE_ROWS_ONE_IN = 16
# workgroups the listed rows are spread over (stretches x blocks of 128 listed rows x batch x heads): about two per slot
_WORKGROUPS_WANTED = 512
# the extra launch, the sum over the stretches and the scatter cost about 30 us: taken when the longest column's walk
# (tiles of 64 queries, times the rounds in which the part runs the blocks of 128 keys) is longer than this many tiles
_WORTH_TILES = 40


def keys_side_schedule(segments_t: ACSRSegments, L: int, device, batch_heads: int,
                       always: bool = False) -> KeysSideSchedule | None:
    """The ``KeysSideSchedule`` of a transposed mask, or None when no segment of it is row-sparse (or all are, or a
    sparse one lacks its rows' first columns, or two of them keep the same key), or when the walk it replaces is too short for the extra launch to pay
    (unless ``always``).  A block of 128 consecutive keys of a strided pattern's far field holds
    one live key with up to L queries: its workgroup walks up to L / 64 tiles for one row in 128, and the pass takes 5 x
    what the rest of the mask needs.  Listed row by row and cut into stretches of queries, the same entries fill a few
    workgroups each.  Built once per (L, device, number of stretches) and kept with ``segments_t`` (a host
    synchronisation the first time: not under stream capture, where None is returned unless the schedule exists)."""
    dev = _hip.resolve_device(device)
    cache = segments_t.__dict__.setdefault("_keys_side", {})
    facts = cache.get(("facts", L, dev.index))
    if facts is None:
        if torch.cuda.is_current_stream_capturing():
            return None
        sparse, first, step, cnt, key = [], [], [], [], []
        for i, (t, fc) in enumerate(zip(segments_t.tuples, segments_t.first_cols)):
            nnz = t[4]
            live = torch.nonzero(nnz[:L] > 0).flatten()
            if fc is None or live.numel() == 0 or live.numel() * _SPARSE_ROWS_ONE_IN > L:
                continue
            sparse.append(i)
            n = nnz[live].to(torch.int64)
            key.append(live)
            first.append(fc[live].to(torch.int64))
            step.append(torch.where(n > 1, t[2][live].to(torch.int64), torch.ones_like(n)).clamp(min=1))
            cnt.append(n)
        if not sparse or len(sparse) == len(segments_t) or torch.cat(key).unique().numel() != sum(x.numel() for x in key):
            facts = False
        else:
            first, step, cnt, key = (torch.cat(x) for x in (first, step, cnt, key))
            last = first + step * (cnt - 1)
            facts = (sparse, first, step, cnt, key, int(first.min()), int(last.max()), int((last - first).max()) // 64 + 1)
        cache[("facts", L, dev.index)] = facts
    if facts is False:
        return None
    sparse, first, step, cnt, key, p_min, p_max, longest_tiles = facts
    rounds = -(-batch_heads * -(-L // 128) // 512)
    if not always and longest_tiles * rounds < _WORTH_TILES:
        return None
    n_keys = key.numel()
    per_stretch = -(-n_keys // 128) * 128
    # stretches: enough workgroups to fill the part about twice, at least 8 tiles of 64 queries each
    span = p_max - p_min + 1
    want = max(1, round(_WORKGROUPS_WANTED / max(1, batch_heads * (per_stretch // 128))))
    n_stretches = max(1, min(want, -(-span // 512)))
    sched = cache.get((L, dev.index, n_stretches))
    if sched is not None:
        return sched
    if torch.cuda.is_current_stream_capturing():
        return None
    width = -(-span // (n_stretches * 64)) * 64
    lo = p_min + width * torch.arange(n_stretches, device=dev, dtype=torch.int64)[:, None]   # [stretches, 1]
    hi = lo + width - 1
    # the entries t of a row (columns first + step * t, t < cnt) that fall into [lo, hi]
    t_lo = torch.div((lo - first[None, :]).clamp(min=0) + step[None, :] - 1, step[None, :], rounding_mode="floor")
    t_hi = torch.minimum(torch.div(hi - first[None, :], step[None, :], rounding_mode="floor"), (cnt - 1)[None, :])
    n = torch.where(hi >= first[None, :], (t_hi - t_lo + 1).clamp(min=0), torch.zeros_like(t_lo))
    f = torch.where(n > 0, first[None, :] + step[None, :] * t_lo, torch.zeros_like(n))

    def padded(x, fill, dtype):
        out = torch.full((n_stretches, per_stretch), fill, dtype=dtype, device=dev)
        out[:, :n_keys] = x.to(dtype)
        return out.flatten().contiguous()
    lin = padded(step[None, :].expand_as(n), 1, torch.float32)
    fcol = padded(f, 0, torch.int32)
    nnz = padded(n, 0, torch.float32)
    trans = (fcol.to(torch.float32) / lin).contiguous()
    rows = ACSRSegments([((1.0 / lin).contiguous(), (-trans).contiguous(), lin, trans, nnz, max(int(n.max()), 1), None, None)],
                        [fcol])
    main = ACSRSegments([t for i, t in enumerate(segments_t.tuples) if i not in sparse],
                        [c for i, c in enumerate(segments_t.first_cols) if i not in sparse])
    key_of_row = padded(key[None, :].expand(n_stretches, n_keys), -1, torch.int32)
    sched = KeysSideSchedule(main, rows, key_of_row, key.contiguous(), n_stretches, per_stretch)
    sched.main.plan(L, dev)
    sched.rows.plan(sched.n_rows, dev)
    cache[(L, dev.index, n_stretches)] = sched
    return sched


def attention_backward_fused(q: torch.Tensor, kT: torch.Tensor, v: torch.Tensor, out: torch.Tensor, grad_out: torch.Tensor,
                             lse: torch.Tensor, segments: ACSRSegments, segments_t: ACSRSegments, plan: torch.Tensor,
                             plan_t: torch.Tensor, scale: float = 1.0, sparse_rows: bool | None = None):
    """(dq, dk, dv) as ``attention_backward`` gives them, from three launches of one kernel and without a compressed
    matrix: ``out`` and ``lse`` are the output and the row statistic of the fused forward for the same inputs
    (``RegularAttention.forward_with_stats``), ``plan`` / ``plan_t`` the fused kernel's plans (``attention_plan``) of the
    mask's segments and of the transposed mask's.  16-bit dtypes, d in {64, 128}; operands whose rows are not contiguous
    16-byte pieces (K^T-contiguous keys among them) are copied first.  Segments of the transposed mask that keep few keys
    with long columns are taken row by row (``keys_side_schedule``; ``plan_t`` then goes unused) where that pays (``sparse_rows`` None), wherever
    there are such segments (True) or never (False)."""
    B, H, L, d = q.shape
    dt, dev = q.dtype, q.device
    if dt not in (torch.float16, torch.bfloat16) or d not in (64, 128):
        raise _hip.SplatError("the fused backward takes fp16 / bf16 tensors with d in {64, 128}")
    # K^T with the keys contiguous (the reference's layout): one streaming transpose instead of a strided copy
    k = transpose_keys(kT) if (kT.dim() == 4 and kT.stride(3) == 1 and kT.stride(2) != 1) else kT.transpose(2, 3)

    def rows(t, name):
        _hip.require_device_tensor(t, name)
        if t.dtype != dt or tuple(t.shape) != (B, H, L, d):
            raise _hip.SplatError(f"{name} must be a {dt} tensor of shape {(B, H, L, d)}, got {t.dtype} {tuple(t.shape)}")
        if t.stride(3) != 1 or t.data_ptr() % 16 != 0 or any(t.stride(i) % 8 != 0 for i in (0, 1, 2)):
            t = t.contiguous()
        return t
    q, k, v, out, grad_out = rows(q, "q"), rows(k, "k"), rows(v, "v"), rows(out, "out"), rows(grad_out, "grad_out")
    _hip.require_device_tensor(lse, "lse")
    if lse.dtype != torch.float32 or tuple(lse.shape) != (B, H, L) or not lse.is_contiguous():
        raise _hip.SplatError(f"lse must be a contiguous float32 tensor of shape {(B, H, L)}")
    delta = torch.empty((B, H, L), dtype=torch.float32, device=dev)
    dq = torch.empty((B, H, L, d), dtype=dt, device=dev)
    dk, dv = (torch.empty((B, H, L, d), dtype=dt, device=dev) for _ in range(2))
    sched = None if sparse_rows is False else keys_side_schedule(segments_t, L, dev, B * H, always=bool(sparse_rows))
    if sched is not None:  # the row-sparse segments of the transposed mask go row by row, after the others
        segments_t, plan_t = sched.main, sched.main.plan(L, dev)
    arr = segments.seg_array(L)
    arr_t = segments_t.seg_array(L)

    def strides3(*tensors):
        a = []
        for t in tensors:
            a += [t.data_ptr(), t.stride(0), t.stride(1), t.stride(2)]
        return a
    args = strides3(q, k, v, out, grad_out)
    args += [lse.data_ptr(), delta.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
             arr, len(segments), plan.data_ptr(), plan.numel() * plan.element_size(),
             arr_t, len(segments_t), plan_t.data_ptr(), plan_t.numel() * plan_t.element_size(),
             B, H, L, d, float(scale), _hip.dtype_code(dt)]
    with torch.cuda.device(dev):
        rc = _hip.lib().splat_attention_bwd(*args, _hip.stream_ptr(dev))
        _hip.check(rc, "splat_attention_bwd")
        if sched is not None:
            R = sched.n_rows
            part = torch.empty((2, B, H, R, d), dtype=dt, device=dev)
            plan_r = sched.rows.plan(R, dev)
            args = strides3(q, k, v, grad_out)
            # (the call's second kernel adds a key's shares, one per stretch, onto what the other segments gave it)
            args += [lse.data_ptr(), delta.data_ptr(), sched.key_of_row.data_ptr(), part[0].data_ptr(), part[1].data_ptr(),
                     sched.rows.seg_array(R), 1, plan_r.data_ptr(), plan_r.numel() * plan_r.element_size(),
                     B, H, L, R, d, float(scale), _hip.dtype_code(dt), dk.data_ptr(), dv.data_ptr(), sched.per_stretch]
            rc = _hip.lib().splat_attention_bwd_keys(*args, _hip.stream_ptr(dev))
            _hip.check(rc, "splat_attention_bwd_keys")
    return dq, dk, dv
