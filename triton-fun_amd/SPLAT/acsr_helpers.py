"""ACSR (affine-compressed sparse row) metadata for SPLAT's regular sparse kernels, built on the GPU.

Mirrors the interface of the reference's ``SPLAT/acsr_helpers.py`` (mask generators :18-55, ACSR
containers :58-96, ``instantiate_metadata`` :99-142, ``create_acsr`` :145-160): same names, same
positional arguments, same return tuples, every metadata tensor float32.  The O(L^2) Python passes of
the reference are replaced by one streaming HIP kernel over a byte mask (``splat_acsr_build``).

Additions that keep the reference behaviour as the default:
  * masks may also be numpy arrays, torch tensors (host or device) or :class:`MaskPattern` descriptors
    that are rasterised on the device, so L = 16384 never needs a Python list of lists;
  * ``create_acsr_segments`` builds several disjoint affine segments per row (e.g. a local window plus
    a strided far field), which one affine map per row cannot express.
"""
from __future__ import annotations

from dataclasses import dataclass
from math import ceil
from typing import Any, Sequence, Type

import hashlib
import weakref

import numpy as np
import torch

import _splat_hip as _hip

# ---------------------------------------------------------------------------------------------
# Mask generators (s = sequence length, p = sparsity parameter); list-of-lists like the reference.
# ---------------------------------------------------------------------------------------------


def _row(s: int, lo: int, hi: int) -> list[int]:
    lo, hi = max(lo, 0), min(hi, s)
    if hi <= lo:
        return [0] * s
    return [0] * lo + [1] * (hi - lo) + [0] * (s - hi)


def create_blocked_mask(s: int, p: int, device: Any = None):
    """Rows of the first block see columns [0, p); row i of a later block sees the previous block and
    its own: [(i//p - 1)*p, (i//p + 1)*p).  With ``device`` set, returns a uint8 tensor rasterised there."""
    if device is not None:
        return MaskPattern(_hip.MASK_BLOCKED, s, p).device_mask(device)
    return [_row(s, 0, p) if i < p else _row(s, (i // p - 1) * p, (i // p + 1) * p) for i in range(s)]


def create_windowed_mask(s: int, p: int, device: Any = None):
    """|i - j| <= p."""
    if device is not None:
        return MaskPattern(_hip.MASK_WINDOWED, s, p).device_mask(device)
    return [_row(s, i - p, i + p + 1) for i in range(s)]


def create_causal_windowed_mask(s: int, p: int, device: Any = None):
    """i - p <= j <= i."""
    if device is not None:
        return MaskPattern(_hip.MASK_CAUSAL_WINDOWED, s, p).device_mask(device)
    return [_row(s, i - p, i + 1) for i in range(s)]


@dataclass(frozen=True)
class MaskPattern:
    """A closed-form s x s mask that is rasterised on the device instead of in Python."""
    kind: int
    s: int
    p0: int
    p1: int = 1

    def device_mask(self, device: Any) -> torch.Tensor:
        dev = _hip.resolve_device(device)
        out = torch.empty((self.s, self.s), dtype=torch.uint8, device=dev)
        with torch.cuda.device(dev):
            rc = _hip.lib().splat_mask_generate(out.data_ptr(), self.s, self.s, self.s, self.kind, self.p0, self.p1,
                                                _hip.stream_ptr(dev))
        _hip.check(rc, "splat_mask_generate")
        return out

    def transposed(self) -> "MaskPattern":
        """The transposed pattern (row j keeps the rows of this pattern that keep column j), itself closed-form."""
        return MaskPattern(self.kind ^ _hip.MASK_TRANSPOSED, self.s, self.p0, self.p1)


def blocked_pattern(s: int, p: int) -> MaskPattern:
    return MaskPattern(_hip.MASK_BLOCKED, s, p)


def windowed_pattern(s: int, p: int) -> MaskPattern:
    return MaskPattern(_hip.MASK_WINDOWED, s, p)


def causal_windowed_pattern(s: int, p: int) -> MaskPattern:
    return MaskPattern(_hip.MASK_CAUSAL_WINDOWED, s, p)


def dilated_pattern(s: int, window: int, dilation: int) -> MaskPattern:
    """Row i sees columns i - window*dilation//2 + dilation*t, t in [0, window), clipped to [0, s)."""
    return MaskPattern(_hip.MASK_DILATED, s, window, dilation)


def strided_patterns(s: int, local: int, stride: int) -> list[MaskPattern]:
    """Sparse-Transformer style rows as two disjoint affine segments: the local causal window
    (i - local, i] and the far columns j <= i - local with j % stride == stride - 1."""
    return [MaskPattern(_hip.MASK_STRIDED_LOCAL, s, local), MaskPattern(_hip.MASK_STRIDED_FAR, s, local, stride)]


# ---------------------------------------------------------------------------------------------
# Host containers, as in the reference.
# ---------------------------------------------------------------------------------------------


@dataclass
class AffineIndices:
    """Dense -> sparse map of one row: slot = linear_transformation * column + translation."""
    linear_transformation: float
    translation: int
    nnz: int


@dataclass
class AffineIndicesInt:
    """Sparse -> dense map of one row: column = linear_transformation * (slot + translation)."""
    linear_transformation: int
    translation: int
    nnz: int


class ACSR:
    def __init__(self, affine_indices: list[Type[AffineIndices]], affine_indices_int: list[Type[AffineIndicesInt]],
                 span_specialised_loop_idxs: list[tuple[int]]):
        self.affine_indices = affine_indices
        self.affine_indices_int = affine_indices_int
        self.span_specialised_loop_idxs = span_specialised_loop_idxs

    def get_dTos_linear_transformations(self) -> list[float]:
        return [x.linear_transformation for x in self.affine_indices]

    def get_sTod_linear_transformations(self) -> list[int]:
        return [x.linear_transformation for x in self.affine_indices_int]

    def get_dTos_translations(self) -> list[float]:
        return [x.translation for x in self.affine_indices]

    def get_sTod_translations(self) -> list[int]:
        return [x.translation for x in self.affine_indices_int]

    def get_nnzs(self) -> list[float]:
        return [x.nnz for x in self.affine_indices]

    def get_span_specialised_data(self) -> list[tuple[int]]:
        return self.span_specialised_loop_idxs


# ---------------------------------------------------------------------------------------------
# Device masks and the GPU builder.
# ---------------------------------------------------------------------------------------------


class _MaskEntry:
    __slots__ = ("key", "owner", "builds")

    def __init__(self, key, owner):
        self.key = key
        self.owner = owner  # weak reference to a tensor mask: while it lives, its storage address cannot be reused
        self.builds = {}

    def alive(self) -> bool:
        return self.owner is None or self.owner() is not None


_MASK_CACHE: list[_MaskEntry] = []
_MASK_CACHE_SIZE = 4


def _host_mask_bytes(mask) -> np.ndarray:
    arr = np.asarray(mask)
    if arr.ndim != 2:
        raise ValueError("mask must be a 2-D 0/1 array")
    if arr.size and (arr.min() < 0 or arr.max() > 255):
        raise ValueError("mask entries must fit in a byte")
    return np.ascontiguousarray(arr, dtype=np.uint8)


def _cache_key(mask, host_bytes: np.ndarray | None = None) -> tuple:
    """What identifies a mask's contents.  Tensors: storage address, version counter (bumped by every in-place
    edit made through the tensor itself; writes through ``.data``, ``.numpy()`` or another alias leave it alone, and a
    mask edited that way needs ``_MASK_CACHE.clear()`` before it is built again), shape, strides, storage offset and
    dtype -- a transposed or offset view of the same storage is another mask.  Patterns: the (frozen) descriptor.  Lists and arrays are mutable without a trace, so they are keyed on a
    digest of their bytes, taken from the uint8 copy that the upload needs anyway."""
    if isinstance(mask, torch.Tensor):
        return ("t", mask.data_ptr(), mask._version, tuple(mask.shape), tuple(mask.stride()), mask.storage_offset(),
                str(mask.dtype), str(mask.device))
    if isinstance(mask, MaskPattern):
        return ("p", mask)
    b = _host_mask_bytes(mask) if host_bytes is None else host_bytes
    return ("h", b.shape, hashlib.blake2b(b.data, digest_size=16).digest())


def _mask_entry(mask, dev: torch.device) -> tuple[_MaskEntry, np.ndarray | None]:
    """The cache entry of ``mask`` on ``dev`` (create_acsr and the three preambles are handed the same mask, as in the
    reference, and share one build) and, for host masks, their uint8 bytes.  Only the small per-row results are kept:
    no rows x cols copy of the mask outlives a build."""
    host = None if isinstance(mask, (torch.Tensor, MaskPattern)) else _host_mask_bytes(mask)
    key = (_cache_key(mask, host), str(dev))
    _MASK_CACHE[:] = [e for e in _MASK_CACHE if e.alive()]
    for e in _MASK_CACHE:
        if e.key == key:
            return e, host
    if isinstance(mask, torch.Tensor) and mask.dim() != 2:
        raise ValueError("mask must be 2-D")
    entry = _MaskEntry(key, weakref.ref(mask) if isinstance(mask, torch.Tensor) else None)
    _MASK_CACHE.append(entry)
    del _MASK_CACHE[:-_MASK_CACHE_SIZE]
    return entry, host


def _device_mask(mask, host: np.ndarray | None, dev: torch.device) -> torch.Tensor | None:
    """uint8 [rows, cols] on ``dev`` with unit column stride; None for a MaskPattern (never rasterised for the builder:
    its rows are known in closed form)."""
    if isinstance(mask, MaskPattern):
        return None
    if isinstance(mask, torch.Tensor):
        dm = mask.to(device=dev, dtype=torch.uint8)
        return dm if dm.stride(1) == 1 else dm.contiguous()
    return torch.from_numpy(host).to(dev)


def mask_shape(mask) -> tuple[int, int]:
    if isinstance(mask, MaskPattern):
        return (mask.s, mask.s)
    if isinstance(mask, torch.Tensor):
        return tuple(mask.shape)
    return (len(mask), len(mask[0]))


class _FromSummary:
    """An integer the builder left on the device (its summary record), read back when somebody asks for its value and
    not before: ``int(x)`` synchronises once, then every figure of the record is known."""
    __slots__ = ("build", "name")

    def __init__(self, build: "AcsrBuild", name: str):
        self.build, self.name = build, name

    def __int__(self) -> int:
        self.build.resolve()
        return getattr(self.build, "_" + self.name)

    __index__ = __int__

    def __repr__(self) -> str:
        return f"<{self.name} of an ACSR build, read back on use>"


class AcsrBuild:
    """Everything one ``splat_acsr_build`` call produced for (mask, BLOCK_HEIGHT).  ``T``, ``row_stride`` and
    ``max_step`` come from a summary record the kernels leave on the device; reading it is the build's only
    synchronisation and happens on first use (``resolve``)."""
    __slots__ = ("dTos_lin", "dTos_trans", "sTod_lin", "sTod_trans", "nnz", "span_start", "span_end",
                 "row_first", "row_last", "summary", "_T", "_row_stride", "_max_step")

    def resolve(self) -> None:
        if self.summary is None:
            return
        found = self.summary.cpu()  # the one synchronisation: T is returned as a Python int, like the reference
        self.summary = None
        assert int(found[1]) == 0, "Incorrect unpacking of affine-indices."
        self._T = int(found[0])
        # rows whose columns step by n and start in phase with the row index (dilated windows): kernels group them by phase
        self._row_stride = int(found[2]) if (int(found[2]) == int(found[3]) and int(found[3]) > 1 and int(found[4]) == 0) else 1
        # the largest column step of any row: above 1 some rows are gathered (dilated windows, strided far fields)
        self._max_step = int(found[3])

    @property
    def T(self) -> int:
        self.resolve()
        return self._T

    @property
    def row_stride(self) -> int:
        self.resolve()
        return self._row_stride

    @property
    def max_step(self) -> int:
        self.resolve()
        return self._max_step


def build_acsr(mask, BLOCK_HEIGHT: int, dev: torch.device) -> AcsrBuild:
    entry, host = _mask_entry(mask, dev)
    if BLOCK_HEIGHT in entry.builds:
        return entry.builds[BLOCK_HEIGHT]
    dm = _device_mask(mask, host, dev)
    rows, cols = mask_shape(mask) if dm is None else dm.shape
    n_blocks = ceil(rows / BLOCK_HEIGHT)
    f32 = dict(dtype=torch.float32, device=dev)
    b = AcsrBuild()
    b.dTos_lin, b.dTos_trans = torch.empty(rows, **f32), torch.empty(rows, **f32)
    b.sTod_lin, b.sTod_trans = torch.empty(rows, **f32), torch.empty(rows, **f32)
    b.nnz = torch.empty(rows, **f32)
    b.span_start, b.span_end = torch.empty(n_blocks, **f32), torch.empty(n_blocks, **f32)
    b.row_first = torch.empty(rows, dtype=torch.int32, device=dev)
    b.row_last = torch.empty(rows, dtype=torch.int32, device=dev)
    b.summary = torch.empty(8, dtype=torch.int32, device=dev)
    outs = (b.dTos_lin.data_ptr(), b.dTos_trans.data_ptr(), b.sTod_lin.data_ptr(), b.sTod_trans.data_ptr(), b.nnz.data_ptr(),
            b.span_start.data_ptr(), b.span_end.data_ptr(), b.row_first.data_ptr(), b.row_last.data_ptr(), b.summary.data_ptr())
    with torch.cuda.device(dev):
        if dm is None:  # a MaskPattern: O(rows) work, no rows x cols buffer
            rc = _hip.lib().splat_acsr_build_pattern(mask.kind, mask.s, mask.p0, mask.p1, BLOCK_HEIGHT, *outs,
                                                     _hip.stream_ptr(dev))
            _hip.check(rc, "splat_acsr_build_pattern")
        else:
            rc = _hip.lib().splat_acsr_build(dm.data_ptr(), rows, cols, dm.stride(0), BLOCK_HEIGHT, *outs,
                                             _hip.stream_ptr(dev))
            _hip.check(rc, "splat_acsr_build")
    entry.builds[BLOCK_HEIGHT] = b
    return b


def instantiate_metadata(mask, BLOCK_HEIGHT: int, GPU_ID: Any = 0) -> ACSR:
    """Host containers of the ACSR (values as stored, i.e. rounded to float32)."""
    b = build_acsr(mask, BLOCK_HEIGHT, _hip.resolve_device(GPU_ID))
    a0, a1 = b.dTos_lin.tolist(), b.dTos_trans.tolist()
    s0, s1 = b.sTod_lin.tolist(), b.sTod_trans.tolist()
    nz = [int(x) for x in b.nnz.tolist()]
    d2s = [AffineIndices(a0[i], a1[i], nz[i]) for i in range(len(nz))]
    s2d = [AffineIndicesInt(int(s0[i]), s1[i], nz[i]) for i in range(len(nz))]
    return ACSR(d2s, s2d, list(zip(b.span_start.tolist(), b.span_end.tolist())))


def create_acsr(mask, BLOCK_HEIGHT: int, GPU_ID: Any, *, T: int | None = None):
    """(dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnzs, T, span_loop_start, span_loop_end): seven float32
    device tensors and the trailing dimension T = max row nnz as an int.

    The reference returns ``T`` as a Python int (acsr_helpers.py:153), which here means reading one word back from the
    device: the call's only synchronisation.  A caller that knows the trailing dimension of its pattern passes it as
    ``T=`` and the call only enqueues work; the builder's own figure (and its assertion on rows it could not solve) are
    then checked when the metadata is first used by a launcher, where a mismatch raises ``SplatError``.

    The returned ``sTod_translations`` tensor carries an attribute ``splat_first_col`` (int32 tensor, first
    live column per row) that the launchers pick up: rows with a single live column store translation 0
    whatever that column is, so the column itself has to travel separately.  ``splat_row_stride`` is a speed
    hint for patterns whose rows alternate column phase, ``splat_max_step`` the largest column step of any row (both
    convert with ``int()``; after a call with ``T=`` that conversion is what reads the builder's record back)."""
    dev = _hip.resolve_device(GPU_ID)
    b = build_acsr(mask, BLOCK_HEIGHT, dev)
    if T is None:
        b.resolve()
    # every caller gets tensors of its own, as from the reference's create_acsr: a build shared through the cache must
    # not change under one caller because another one wrote into its metadata
    arrays = [t.clone() for t in (b.dTos_lin, b.dTos_trans, b.sTod_lin, b.sTod_trans, b.nnz, b.span_start, b.span_end)]
    arrays[3].splat_first_col = b.row_first.clone()
    if b.summary is None:
        if T is not None and int(T) != b.T:
            raise _hip.SplatError(f"T={T} was given, the mask's longest row has {b.T} live columns")
        arrays[3].splat_row_stride = b.row_stride
        arrays[3].splat_max_step = b.max_step
        t_out = b.T
    else:
        arrays[3].splat_row_stride = _CheckedHint(b, "row_stride", int(T))
        arrays[3].splat_max_step = _CheckedHint(b, "max_step", int(T))
        t_out = int(T)
    return (arrays[0], arrays[1], arrays[2], arrays[3], arrays[4], t_out, arrays[5], arrays[6])


class _CheckedHint(_FromSummary):
    """A hint of a build whose trailing dimension the caller supplied: reading it also compares that figure with the
    builder's."""
    __slots__ = ("claimed_T",)

    def __init__(self, build: AcsrBuild, name: str, claimed_T: int):
        super().__init__(build, name)
        self.claimed_T = claimed_T

    def __int__(self) -> int:
        if self.build.T != self.claimed_T:
            raise _hip.SplatError(f"create_acsr was given T={self.claimed_T}, the mask's longest row has {self.build.T} live columns")
        return super().__int__()

    __index__ = __int__


def transpose_keys(kT: torch.Tensor) -> torch.Tensor:
    """K [B, H, L, d] (contiguous, new) from K^T [B, H, d, L] with unit stride along the keys: one streaming kernel."""
    _hip.require_device_tensor(kT, "kT")
    if kT.dim() != 4 or kT.stride(3) != 1:
        raise _hip.SplatError("kT must be [B, H, d, L] with unit stride along the keys")
    B, H, d, L = kT.shape
    out = torch.empty((B, H, L, d), dtype=kT.dtype, device=kT.device)
    if out.numel() == 0:
        return out
    with torch.cuda.device(kT.device):
        rc = _hip.lib().splat_transpose_keys(kT.data_ptr(), kT.stride(0), kT.stride(1), kT.stride(2), out.data_ptr(), B, H, L, d,
                                             _hip.dtype_code(kT.dtype), _hip.stream_ptr(kT.device))
    _hip.check(rc, "splat_transpose_keys")
    return out


class ACSRSegments:
    """Several disjoint affine segments per row.  Segment k owns compressed slots
    [offsets[k], offsets[k] + T_k); ``T`` is the total trailing dimension."""

    def __init__(self, tuples: Sequence[tuple], first_cols: Sequence[torch.Tensor | None]):
        # a segment that is empty in every row (trailing dimension 0) owns no slots: it is dropped, unless it is all
        # there is (its slot offset would equal the row length, which the kernels reject)
        keep = [i for i, t in enumerate(tuples) if int(t[5]) > 0] or [0]
        self.tuples = [tuples[i] for i in keep]
        self.first_cols = [first_cols[i] for i in keep]
        self.offsets = []
        off = 0
        for t in self.tuples:
            self.offsets.append(off)
            off += int(t[5])
        self.T = off
        self._plan_holder = None  # where plan() keeps its tables when not with this object
        self._arrays = {}  # seg_array()'s results

    def __len__(self) -> int:
        return len(self.tuples)

    @property
    def max_step(self) -> int:
        """The largest column step of any row of any segment (1 when unknown: metadata not built by ``create_acsr``)."""
        return max(int(getattr(t[3], "splat_max_step", 1)) for t in self.tuples)

    @property
    def gathered(self) -> bool:
        """Some row of some segment steps over columns."""
        return self.max_step > 1

    def keys_as_rows(self, kT: torch.Tensor, min_step: int = 2) -> torch.Tensor:
        """``kT`` ([B, H, d, L]) as the kernels should get it.  The reference stores K^T contiguously along the keys;
        the kernels read that layout in dense runs of keys, which for gathered rows (every second key of a dilated
        window, every 128th of a strided far field) means walking, and masking, all the keys in between.  With rows
        of K contiguous they fetch only the keys a tile needs, so for masks whose rows step by ``min_step`` columns or
        more K is transposed once per call (its bytes read and written once) and handed on as a [B, H, d, L] view of
        the [B, H, L, d] copy."""
        if self.max_step >= min_step and kT.dim() == 4 and kT.stride(3) == 1 and kT.stride(2) != 1:
            return transpose_keys(kT).transpose(2, 3)
        return kT

    def plan(self, L: int, device) -> torch.Tensor:
        """The plan table of these segments for ``L`` rows (``splat_attention_plan``: which key tiles each 128-row block
        walks, every row's window), built on first use and kept: with the segments themselves, or, for metadata that
        came in as separate tensors, with its ``sTod_translations`` tensor (attribute ``splat_plans``), so that the
        next launcher call with the same tensors finds it.  The metadata is taken to be immutable from then on."""
        dev = _hip.resolve_device(device)
        holder = self._plan_holder if self._plan_holder is not None else self
        plans = getattr(holder, "splat_plans", None)
        if plans is None:
            plans = {}
            holder.splat_plans = plans
        key = (int(L), len(self), tuple(self.offsets), dev.index)
        if key not in plans:
            arr = self.seg_array(L)
            nbytes = int(_hip.lib().splat_attention_plan_bytes(arr, len(self), L))
            if nbytes <= 0:
                raise _hip.SplatError(f"no plan for {len(self)} segments and L={L}")
            table = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            with torch.cuda.device(dev):
                rc = _hip.lib().splat_attention_plan(arr, len(self), L, table.data_ptr(), nbytes, _hip.stream_ptr(dev))
                _hip.check(rc, "splat_attention_plan")
                # once, so that later launches may run on any stream without ordering themselves after the plan kernel
                torch.cuda.current_stream(dev).synchronize()
                # whether every live row starts on a multiple of 8 positions of its block's walk (blocked masks): one look
                # at the rows' records of the first variant (gathered walks), which follow its 5 records per block and
                # segment: [lo, cnt, lin, phase] each
                n_rb = nbytes // (2 * len(self) * (5 + 128) * 16)
                recs = table.view(torch.int32).view(-1, 4)
                rows = recs[n_rb * len(self) * 5:n_rb * len(self) * (5 + 128)]
                aligned = bool((((rows[:, 0] & 7) == 0) | (rows[:, 1] <= 0)).all())
            plans[key] = (table, aligned)
        return plans[key][0]

    def has_plan(self, L: int, device) -> bool:
        """Whether ``plan`` would return a table it already holds (no kernel, no synchronisation)."""
        dev = _hip.resolve_device(device)
        holder = self._plan_holder if self._plan_holder is not None else self
        return (int(L), len(self), tuple(self.offsets), dev.index) in getattr(holder, "splat_plans", {})

    def plan_is_aligned(self, L: int, device) -> bool:
        """Whether every row of the plan for ``L`` rows starts on a multiple of 8 positions (see ``plan``)."""
        self.plan(L, device)
        holder = self._plan_holder if self._plan_holder is not None else self
        dev = _hip.resolve_device(device)
        return holder.splat_plans[(int(L), len(self), tuple(self.offsets), dev.index)][1]

    def seg_args(self) -> list[tuple]:
        return [(t[0], t[1], t[2], t[3], t[4], fc, off) for t, fc, off in zip(self.tuples, self.first_cols, self.offsets)]

    def seg_array(self, rows: int, trailing_dim: int | None = None):
        """The segments as the C ABI takes them (``_splat_hip.seg_array``), checked and built once per (rows, trailing
        dimension) and kept: the metadata is taken to be immutable, and its tensors live as long as this object."""
        key = (int(rows), None if trailing_dim is None else int(trailing_dim))
        arr = self._arrays.get(key)
        if arr is None:
            arr = self._arrays[key] = _hip.seg_array(self.seg_args(), rows, trailing_dim)
        return arr

    @staticmethod
    def single(dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnzs, T) -> "ACSRSegments":
        fc = getattr(sTod_trans, "splat_first_col", None)
        segs = ACSRSegments([(dTos_lin, dTos_trans, sTod_lin, sTod_trans, nnzs, T, None, None)], [fc])
        segs._plan_holder = sTod_trans
        return segs


def create_acsr_segments(masks: Sequence, BLOCK_HEIGHT: int, GPU_ID: Any) -> ACSRSegments:
    """One ``create_acsr`` per segment mask; the masks must be pairwise disjoint."""
    tuples = [create_acsr(m, BLOCK_HEIGHT, GPU_ID) for m in masks]
    return ACSRSegments(tuples, [t[3].splat_first_col for t in tuples])


def non_affine_rows(mask_u8: torch.Tensor, row_first: torch.Tensor, sTod_lin: torch.Tensor, nnz: torch.Tensor,
                    chunk_rows: int = 2048) -> torch.Tensor:
    """Indices (int64, on the mask's device) of the rows of a 0/1 byte mask whose live columns are not the arithmetic
    progression ``first + step * t, t < nnz`` that the row's metadata stands for (``instantiate_metadata`` takes the step
    from the first two live columns only, acsr_helpers.py:112-124, and nothing in the reference looks at the rest of the
    row).  A row passes when all of its ``nnz`` ones sit on the progression's ``nnz`` positions, which makes the two sets
    equal.  Plain tensor code, so it runs on host tensors as well."""
    rows, cols = mask_u8.shape
    n = nnz.to(torch.int64)
    step = sTod_lin.to(torch.int64).clamp(min=1)
    first = row_first.to(torch.int64)
    bad = []
    width = int(n.max()) if rows else 0
    t = torch.arange(max(width, 1), device=mask_u8.device, dtype=torch.int64)[None, :]
    for r0 in range(0, rows, chunk_rows):
        r1 = min(rows, r0 + chunk_rows)
        pos = first[r0:r1, None] + step[r0:r1, None] * t
        live = t < n[r0:r1, None]
        inside = live & (pos >= 0) & (pos < cols)
        hits = (mask_u8[r0:r1].gather(1, pos.clamp(0, cols - 1)).to(torch.int64) * inside).sum(1)
        bad.append(torch.nonzero(hits != n[r0:r1]).flatten() + r0)
    return torch.cat(bad) if bad else torch.empty(0, dtype=torch.int64, device=mask_u8.device)


def row_extents(mask, GPU_ID: Any) -> tuple[torch.Tensor, torch.Tensor]:
    """(first, last) nonzero column per row as int32 device tensors (cols / -1 for an empty row)."""
    b = build_acsr(mask, 16, _hip.resolve_device(GPU_ID))
    return b.row_first, b.row_last
