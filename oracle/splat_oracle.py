"""CPU restatement of SPLAT's ACSR sparse-attention path.  TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels: only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import it.  Nothing under the product package
imports, calls or falls back to it.

Every function cites the reference lines (under ``SPLAT/``) it restates.  The reference's Triton
kernels are known to be wrong outside a narrow envelope (softmax touches only L/BLOCK rows,
SpMM write-back mask swaps m/n, ...), so for the numeric operators the oracle restates the
*checker* the reference itself uses (``truth`` einsum, ``dot_product``, row-sum == 1) and the
dense masked attention those checkers imply, not the kernels.

Pinning status (what independent evidence each function is checked against in ``tests/``):
  * mask generators ........ literal known-answer matrices + closed-form row sums
  * instantiate_metadata ... hand-derived known answers (blocked 10/2, an irregular row),
                             closed forms per pattern, slot->column round trip against the mask,
                             brute-force float32(solve) == float32(closed form)
  * naive_block_mappings ... hand-derived known answers on tiny masks
  * numeric operators ...... textbook definitions (einsum / softmax / matmul) cross-checked
                             against each other through compress/decompress identities
No function here is "parity unpinned".
"""
from __future__ import annotations

from math import ceil, log2

import numpy as np
import torch

# ----------------------------------------------------------------------------------------------
# Masks.  Reference: acsr_helpers.py:18-55.  Returned as uint8 [s, s] arrays (``.tolist()`` gives
# the reference's list-of-lists).
# ----------------------------------------------------------------------------------------------


def create_blocked_mask(s: int, p: int) -> np.ndarray:
    """acsr_helpers.py:18-34: rows < p see columns < p; row i >= p sees
    [(i//p - 1)*p, (i//p - 1)*p + 2p)."""
    i = np.arange(s)[:, None]
    j = np.arange(s)[None, :]
    start = (i // p - 1) * p
    later = (i >= p) & (start <= j) & (j < start + 2 * p)
    first = (i < p) & (j < p)
    return (first | later).astype(np.uint8)


def create_windowed_mask(s: int, p: int) -> np.ndarray:
    """acsr_helpers.py:36-44: |i - j| <= p."""
    i = np.arange(s)[:, None]
    j = np.arange(s)[None, :]
    return ((i - p <= j) & (j <= i + p)).astype(np.uint8)


def create_causal_windowed_mask(s: int, p: int) -> np.ndarray:
    """acsr_helpers.py:46-55: i - p <= j <= i."""
    i = np.arange(s)[:, None]
    j = np.arange(s)[None, :]
    return ((i - p <= j) & (j <= i + p) & (i >= j)).astype(np.uint8)


def create_dilated_mask(s: int, window: int, dilation: int) -> np.ndarray:
    """Benchmark pattern (not in the reference): row i sees columns i - window*dilation/2 + dilation*t,
    t in [0, window), clipped to [0, s).  window=512, dilation=2 gives i-512, i-510, ..., i+510."""
    i = np.arange(s)[:, None]
    j = np.arange(s)[None, :]
    lo = i - (window * dilation) // 2
    rel = j - lo
    return ((rel >= 0) & (rel < window * dilation) & (rel % dilation == 0)).astype(np.uint8)


def create_strided_segment_masks(s: int, local: int, stride: int) -> list[np.ndarray]:
    """Benchmark pattern (not in the reference), Sparse-Transformer style, as two disjoint affine
    segments: [0] local causal window of ``local`` columns (i-local+1 .. i); [1] the columns
    j <= i - local with j % stride == stride - 1."""
    i = np.arange(s)[:, None]
    j = np.arange(s)[None, :]
    seg_local = ((j <= i) & (j > i - local)).astype(np.uint8)
    seg_strided = ((j <= i - local) & (j % stride == stride - 1)).astype(np.uint8)
    return [seg_local, seg_strided]


# ----------------------------------------------------------------------------------------------
# ACSR metadata.  Reference: acsr_helpers.py:99-160.
# ----------------------------------------------------------------------------------------------


def _first_two_ones(mask: np.ndarray):
    """Columns of the first two entries equal to 1 in each row (-1 when absent);
    acsr_helpers.py:112-117 tests ``col == 1``."""
    ones = mask == 1
    cols = mask.shape[1]
    idx = np.where(ones, np.arange(cols)[None, :], cols)
    a = idx.min(axis=1)
    idx2 = np.where(idx == a[:, None], cols, idx)
    b = idx2.min(axis=1)
    a = np.where(a == cols, -1, a)
    b = np.where(b == cols, -1, b)
    return a.astype(np.int64), b.astype(np.int64)


def instantiate_metadata(mask, BLOCK_HEIGHT: int) -> dict:
    """acsr_helpers.py:99-142, vectorised.  Returns float64/int host values exactly as the
    reference holds them before the float32 tensor conversion:
      dTos_lin/dTos_trans ... np.linalg.solve([[a,1],[b,1]], [0,1]) per row with nnz > 1  (:122)
      sTod_lin = round(1/x0), sTod_trans = abs(x1)                                        (:124)
      rows with nnz <= 1 -> (1, 0) / (1, 0)                                               (:126-130)
      span[g] = (min(start, sTod_trans), max(end, nnz*sTod_lin + sTod_trans)), init (cols, -1) (:103,:135-140)
    """
    mask = np.asarray(mask)
    rows, cols = mask.shape
    nnz = mask.astype(np.int64).sum(axis=1)  # reduce(+) over the row (:110)
    a, b = _first_two_ones(mask)
    multi = nnz > 1
    if np.any(multi & ((a == -1) | (b == -1))):
        raise AssertionError("Incorrect unpacking of affine-indices.")  # (:119)

    x0 = np.ones(rows, dtype=np.float64)
    x1 = np.zeros(rows, dtype=np.float64)
    if multi.any():
        am = a[multi].astype(np.int64)
        bm = b[multi].astype(np.int64)
        A = np.empty((am.size, 2, 2), dtype=np.int64)
        A[:, 0, 0] = am
        A[:, 0, 1] = 1
        A[:, 1, 0] = bm
        A[:, 1, 1] = 1
        rhs = np.broadcast_to(np.array([0, 1], dtype=np.int64), (am.size, 2))[..., None]
        sol = np.linalg.solve(A, rhs)[..., 0]
        x0[multi] = sol[:, 0]
        x1[multi] = sol[:, 1]
    sTod_lin = np.rint(1.0 / x0).astype(np.int64)  # Python round() of a float: half-to-even, as rint
    sTod_trans = np.abs(x1)

    n_blocks = ceil(rows / BLOCK_HEIGHT)
    span_start = np.full(n_blocks, float(cols), dtype=np.float64)
    span_end = np.full(n_blocks, -1.0, dtype=np.float64)
    g = np.arange(rows) // BLOCK_HEIGHT
    np.minimum.at(span_start, g, sTod_trans)
    np.maximum.at(span_end, g, nnz * sTod_lin + sTod_trans)
    return dict(dTos_lin=x0, dTos_trans=x1, sTod_lin=sTod_lin, sTod_trans=sTod_trans, nnz=nnz,
                span_start=span_start, span_end=span_end, first=a, second=b)


def instantiate_metadata_rowwise(mask, BLOCK_HEIGHT: int) -> dict:
    """The same as :func:`instantiate_metadata` written as the reference's per-row Python loop
    (acsr_helpers.py:107-140), one ``np.linalg.solve`` call per row.  Small inputs only; used to
    show the vectorised form changes nothing."""
    mask = [list(map(int, row)) for row in np.asarray(mask).tolist()]
    rows, cols = len(mask), len(mask[0])
    out = dict(dTos_lin=[], dTos_trans=[], sTod_lin=[], sTod_trans=[], nnz=[])
    span = [(cols, -1) for _ in range(ceil(rows / BLOCK_HEIGHT))]
    for r in range(rows):
        a = b = -1
        nnz = sum(mask[r])
        if nnz > 1:
            for idx, col in enumerate(mask[r]):
                if col == 1 and a == -1:
                    a = idx
                elif col == 1 and a != -1 and b == -1:
                    b = idx
                    break
            assert a != -1 and b != -1, "Incorrect unpacking of affine-indices."
            x = np.linalg.solve(np.array([[a, 1], [b, 1]]), np.array([0, 1]))
        else:
            x = (1, 0)
        out["dTos_lin"].append(x[0])
        out["dTos_trans"].append(x[1])
        out["sTod_lin"].append(round(1 / x[0]))
        out["sTod_trans"].append(abs(x[1]))
        out["nnz"].append(nnz)
        s0, s1 = span[r // BLOCK_HEIGHT]
        span[r // BLOCK_HEIGHT] = (min(s0, abs(x[1])), max(s1, nnz * round(1 / x[0]) + abs(x[1])))
    out["span_start"] = [s[0] for s in span]
    out["span_end"] = [s[1] for s in span]
    return out


def create_acsr(mask, BLOCK_HEIGHT: int):
    """acsr_helpers.py:145-160 with the device upload left out: the 8-tuple
    (dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnzs, T, span_start, span_end); every array is
    float32 (torch.FloatTensor / torch.Tensor of a Python list rounds float64 -> float32, :148-156)
    and T = max row sum (:153)."""
    md = instantiate_metadata(mask, BLOCK_HEIGHT)
    f32 = lambda x: np.asarray(x, dtype=np.float64).astype(np.float32)
    T = int(md["nnz"].max()) if md["nnz"].size else 0
    return (f32(md["dTos_lin"]), f32(md["dTos_trans"]), f32(md["sTod_lin"]), f32(md["sTod_trans"]),
            f32(md["nnz"]), T, f32(md["span_start"]), f32(md["span_end"]))


def row_extents(mask) -> tuple[np.ndarray, np.ndarray]:
    """First and last truthy column of each row (cols / -1 when the row is empty)."""
    mask = np.asarray(mask) != 0
    cols = mask.shape[1]
    idx = np.arange(cols)[None, :]
    first = np.where(mask, idx, cols).min(axis=1)
    last = np.where(mask, idx, -1).max(axis=1)
    return first.astype(np.int32), last.astype(np.int32)


# ----------------------------------------------------------------------------------------------
# Thread-block anchor maps and preamble bookkeeping.  Reference: r_sddmm.py:117-169,
# r_softmax.py:108-124, r_spmm.py:128-145.
# ----------------------------------------------------------------------------------------------


def naive_block_mappings(mask, BLOCK_HEIGHT: int, BLOCK_WIDTH: int):
    """r_sddmm.py:117-146, quirks kept: only max(rows // BLOCK_HEIGHT, 1) row blocks are visited
    (:124), anchors run ``while x < max_col`` from min_col in steps of BLOCK_WIDTH (:139-142), so a
    block whose nonzeros sit in one column yields no anchor; no anchors at all -> AssertionError."""
    mask = np.asarray(mask) != 0
    rows, cols = mask.shape
    xs: list[int] = []
    ys: list[int] = []
    for blk in range(max(rows // BLOCK_HEIGHT, 1)):
        sub = mask[blk * BLOCK_HEIGHT:(blk + 1) * BLOCK_HEIGHT]
        nz = np.nonzero(sub.any(axis=0))[0]
        lo, hi = (int(nz[0]), int(nz[-1])) if nz.size else (cols, 0)
        x = lo
        while x < hi:
            xs.append(x)
            ys.append(blk * BLOCK_HEIGHT)
            x += BLOCK_WIDTH
    assert len(xs) == len(ys) and len(xs) > 0, "Issues with generating arrangement!"
    return np.asarray(xs, dtype=np.int32), np.asarray(ys, dtype=np.int32)


def rsddmm_grid(n_tiles: int, output_shape) -> tuple[int, int]:
    """r_sddmm.py:165."""
    return (n_tiles, output_shape[0] * output_shape[1])


def rsoftmax_pow2(T: int) -> int:
    """r_softmax.py:112."""
    return 2 ** ceil(log2(T))


def rsoftmax_grid(rows: int, BLOCK_SIZE_X: int, output_shape) -> tuple[int, int]:
    """r_softmax.py:120."""
    return (-(-rows // BLOCK_SIZE_X), output_shape[0] * output_shape[1])


def rspmm_grid(output_shape, BLOCK_SIZE_X: int, BLOCK_SIZE_Y: int) -> tuple[int, int, int]:
    """r_spmm.py:141."""
    return (-(-output_shape[3] // BLOCK_SIZE_X), -(-output_shape[2] // BLOCK_SIZE_Y),
            output_shape[0] * output_shape[1])


# ----------------------------------------------------------------------------------------------
# Compressed layout.  Slot s of row r holds dense column c = sTod_lin[r] * (s + sTod_trans[r])
# (the builder's own definition, acsr_helpers.py:122-124; equals the checkers'
# round(s*lin + trans) at r_sddmm.py:210 / r_spmm.py:187 whenever lin == 1).
# ----------------------------------------------------------------------------------------------


def slot_columns(acsr, T: int | None = None, first_col=None) -> tuple[np.ndarray, np.ndarray]:
    """(cols [rows, T] int64, valid [rows, T] bool).  ``first_col`` (optional, per row) overrides
    the column of slot 0 for rows with exactly one nonzero, whose stored translation the reference
    hard-codes to 0 (acsr_helpers.py:126-130)."""
    sTod_lin = np.asarray(acsr[2], dtype=np.float64)
    sTod_trans = np.asarray(acsr[3], dtype=np.float64)
    nnz = np.asarray(acsr[4], dtype=np.float64)
    T = int(acsr[5]) if T is None else T
    s = np.arange(T, dtype=np.float64)[None, :]
    cols = np.rint(sTod_lin[:, None] * (s + sTod_trans[:, None])).astype(np.int64)
    if first_col is not None:
        single = nnz == 1
        cols[single, 0] = np.asarray(first_col)[single]
    valid = s < nnz[:, None]
    return cols, valid


def compress(dense: torch.Tensor, acsr, first_col=None, fill: float = 0.0) -> torch.Tensor:
    """Gather a dense [..., rows, cols] tensor into compressed [..., rows, T]; dead slots = fill."""
    cols, valid = slot_columns(acsr, first_col=first_col)
    idx = torch.from_numpy(np.where(valid, cols, 0)).to(dense.device)
    out = torch.gather(dense, -1, idx.expand(*dense.shape[:-1], idx.shape[-1]))
    v = torch.from_numpy(valid).to(dense.device)
    return torch.where(v, out, torch.full_like(out, fill))


def decompress(comp: torch.Tensor, acsr, n_cols: int, first_col=None, fill: float = 0.0) -> torch.Tensor:
    """Scatter compressed [..., rows, T] back to dense [..., rows, n_cols]."""
    cols, valid = slot_columns(acsr, T=comp.shape[-1], first_col=first_col)
    dense = torch.full((*comp.shape[:-1], n_cols + 1), fill, dtype=comp.dtype)
    idx = torch.from_numpy(np.where(valid, cols, n_cols))
    dense.scatter_(-1, idx.expand(*comp.shape[:-1], idx.shape[-1]), comp)
    return dense[..., :n_cols]


# ----------------------------------------------------------------------------------------------
# Numeric operators, fp32 on the host.
# ----------------------------------------------------------------------------------------------


def truth(x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """r_sddmm.py:186-188: dense Q.K^T; x [B,H,L,d], y = K^T [B,H,d,L]."""
    return torch.einsum("bnqd,bndk->bnqk", x.float(), y.float())


def sddmm(x, y, acsr, scale: float = 1.0, first_col=None) -> torch.Tensor:
    """What r_sddmm.is_correct accepts (r_sddmm.py:191-221): compressed slot (r, s) equals
    truth[r, c(r, s)] for s < nnz[r]; dead slots returned as 0."""
    return compress(truth(x, y) * scale, acsr, first_col=first_col)


def softmax_compressed(x: torch.Tensor, nnz_slots: torch.Tensor) -> torch.Tensor:
    """r_softmax.py:43-59 intent: per row, softmax over the live slots; dead slots returned as 0.
    ``nnz_slots`` is a bool [rows, T] validity map (several segments may be live in one row)."""
    xf = x.float().masked_fill(~nnz_slots, float("-inf"))
    m = xf.amax(dim=-1, keepdim=True)
    m = torch.where(torch.isfinite(m), m, torch.zeros_like(m))
    e = torch.exp(xf - m)
    s = e.sum(dim=-1, keepdim=True)
    return torch.where(s > 0, e / s, torch.zeros_like(e))


def spmm(p: torch.Tensor, v: torch.Tensor, acsr, first_col=None) -> torch.Tensor:
    """r_spmm.py:183-190 (``dot_product``): out[r, :] = sum_{s < nnz[r]} p[r, s] * v[c(r, s), :]."""
    cols, valid = slot_columns(acsr, T=p.shape[-1], first_col=first_col)
    pd = torch.where(torch.from_numpy(valid), p.float(), torch.zeros((), dtype=torch.float32))
    dense = decompress(pd, acsr, v.shape[-2], first_col=first_col)
    return dense @ v.float()


def dense_masked_attention(q, kT, v, mask, scale: float = 1.0) -> torch.Tensor:
    """fp32 softmax(where(mask, q @ kT * scale, -inf)) @ v.  Rows with no live column give 0.
    ``mask`` is a [L, L] array (any nonzero = live); several segments are passed OR-ed."""
    m = torch.as_tensor(np.asarray(mask) != 0)
    s = truth(q, kT) * scale
    s = s.masked_fill(~m, float("-inf"))
    mx = s.amax(dim=-1, keepdim=True)
    mx = torch.where(torch.isfinite(mx), mx, torch.zeros_like(mx))
    e = torch.exp(s - mx)
    den = e.sum(dim=-1, keepdim=True)
    p = torch.where(den > 0, e / den, torch.zeros_like(e))
    return p @ v.float()


def dense_masked_attention_chunked(q, kT, v, mask_fn, scale: float, row_chunk: int = 1024) -> torch.Tensor:
    """Same result as :func:`dense_masked_attention`, one (b, h, row chunk) at a time so that the
    fp32 score slab stays small.  ``mask_fn(r0, r1)`` returns the bool mask rows [r0, r1)."""
    B, H, L, d = q.shape
    out = torch.empty(B, H, L, v.shape[-1], dtype=torch.float32)
    for r0 in range(0, L, row_chunk):
        r1 = min(L, r0 + row_chunk)
        m = torch.as_tensor(mask_fn(r0, r1))
        s = torch.matmul(q[:, :, r0:r1].float(), kT.float()) * scale
        s = s.masked_fill(~m, float("-inf"))
        mx = s.amax(dim=-1, keepdim=True)
        mx = torch.where(torch.isfinite(mx), mx, torch.zeros_like(mx))
        e = torch.exp(s - mx)
        den = e.sum(dim=-1, keepdim=True)
        p = torch.where(den > 0, e / den, torch.zeros_like(e))
        out[:, :, r0:r1] = p @ v.float()
    return out


def make_inputs(cfg_seed: int, B: int, H: int, L: int, d: int, dtype: torch.dtype, mul: float = 1.0):
    """Seeded q, k, v ~ N(0,1)*mul drawn in fp32 on the host in that order, then cast."""
    g = torch.Generator("cpu").manual_seed(cfg_seed)
    q = torch.randn(B, H, L, d, generator=g, dtype=torch.float32) * mul
    k = torch.randn(B, H, L, d, generator=g, dtype=torch.float32) * mul
    v = torch.randn(B, H, L, d, generator=g, dtype=torch.float32) * mul
    return q.to(dtype), k.to(dtype), v.to(dtype)


# ----------------------------------------------------------------------------------------------
# Backward pass.  The reference has none (r_attention.py:77-100 is forward only); these are the textbook gradients of
# dense masked attention, in two independent forms that tests/test_oracle_numerics.py checks against each other and
# against finite differences.
# ----------------------------------------------------------------------------------------------


def dense_masked_attention_grads(q, kT, v, mask, scale: float, grad_out):
    """(dq, dk, dv) by reverse-mode differentiation of :func:`dense_masked_attention` in fp32."""
    q32 = q.detach().float().requires_grad_(True)
    k32 = kT.detach().float().transpose(2, 3).contiguous().requires_grad_(True)
    v32 = v.detach().float().requires_grad_(True)
    out = dense_masked_attention(q32, k32.transpose(2, 3), v32, mask, scale)
    out.backward(grad_out.float())
    return q32.grad, k32.grad, v32.grad


def dense_masked_attention_grads_explicit(q, kT, v, mask, scale: float, grad_out):
    """The same gradients from the closed formulas: dV = P^T dO, dP = dO V^T, dS = P o (dP - rowsum(P o dP)) * scale,
    dQ = dS K, dK = dS^T Q."""
    m = torch.as_tensor(np.asarray(mask) != 0)
    q32, k32, v32, g = q.float(), kT.float().transpose(2, 3), v.float(), grad_out.float()
    s = (q32 @ k32.transpose(2, 3)) * scale
    s = s.masked_fill(~m, float("-inf"))
    mx = s.amax(dim=-1, keepdim=True)
    mx = torch.where(torch.isfinite(mx), mx, torch.zeros_like(mx))
    e = torch.exp(s - mx)
    den = e.sum(dim=-1, keepdim=True)
    p = torch.where(den > 0, e / den, torch.zeros_like(e))
    dv = p.transpose(2, 3) @ g
    dp = g @ v32.transpose(2, 3)
    ds = p * (dp - (p * dp).sum(dim=-1, keepdim=True)) * scale
    return ds @ k32, ds.transpose(2, 3) @ q32, dv
