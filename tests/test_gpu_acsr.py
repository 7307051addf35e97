"""GPU ACSR builder, mask rasteriser and tile anchor maps against the oracle: float32 metadata must be
bit-identical (compared as uint32), index arrays equal."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O
import acsr_helpers as A
import r_sddmm
import r_softmax
import r_spmm

pytestmark = pytest.mark.gpu


def bits(t):
    if isinstance(t, torch.Tensor):
        t = t.cpu().numpy()
    return np.asarray(t, dtype=np.float32).view(np.uint32)


def check_acsr(mask, BH, dev):
    got = A.create_acsr(mask, BH, dev)
    arr = mask.cpu().numpy() if isinstance(mask, torch.Tensor) else np.asarray(mask)
    want = O.create_acsr(arr, BH)
    names = ["dTos_lin", "dTos_trans", "sTod_lin", "sTod_trans", "nnz", "T", "span_start", "span_end"]
    for k, name in enumerate(names):
        if k == 5:
            assert got[5] == want[5], name
        else:
            assert got[k].dtype == torch.float32 and got[k].device.type == "cuda"
            assert np.array_equal(bits(got[k]), bits(want[k])), name
    first, last = O.row_extents(arr)
    assert np.array_equal(got[3].splat_first_col.cpu().numpy(), first)
    return got


# the reference's own test masks (r_sddmm.py:264-470): create_blocked_mask(n, p)
REF_BLOCKED = [(10, 2), (10, 5), (10, 7), (16, 5), (16, 16), (32, 10), (32, 20), (32, 32), (128, 57), (1024, 256),
               (1024, 328), (1024, 512)]


@pytest.mark.parametrize("n,p", REF_BLOCKED)
@pytest.mark.parametrize("BH", [2, 16])
def test_blocked_masks_bit_exact(dev, n, p, BH):
    check_acsr(O.create_blocked_mask(n, p), BH, dev)


@pytest.mark.parametrize("make", [
    lambda: O.create_windowed_mask(64, 7), lambda: O.create_windowed_mask(128, 16),
    lambda: O.create_causal_windowed_mask(512, 63), lambda: O.create_causal_windowed_mask(4096, 255),
    lambda: O.create_dilated_mask(2048, 512, 2), lambda: O.create_dilated_mask(300, 16, 3),
    lambda: O.create_strided_segment_masks(1024, 128, 128)[0], lambda: O.create_strided_segment_masks(1024, 128, 128)[1],
    lambda: O.create_causal_windowed_mask(1000, 37),  # row pitch not a multiple of 16: byte path
    lambda: np.eye(33, dtype=np.uint8), lambda: np.zeros((20, 40), np.uint8), lambda: np.ones((40, 20), np.uint8)])
def test_pattern_masks_bit_exact(dev, make):
    check_acsr(make(), 16, dev)


def test_list_of_lists_and_irregular_rows(dev):
    check_acsr(A.create_blocked_mask(10, 2), 2, dev)  # the reference's argument type
    m = np.zeros((3, 10), np.uint8)
    m[0, [3, 7, 8]] = 1
    m[1, 5] = 1
    got = check_acsr(m, 2, dev)
    assert got[0].tolist() == [0.25, 1.0, 1.0] and got[3].tolist() == [0.75, 0.0, 0.0]
    rng = np.random.default_rng(0)
    for _ in range(5):  # arbitrary (non-affine) rows: only the first two ones matter
        check_acsr((rng.random((70, 130)) < 0.1).astype(np.uint8), 16, dev)


def test_assertion_is_kept(dev):
    m = np.zeros((2, 4), np.uint8)
    m[0, 1] = 2
    with pytest.raises(AssertionError, match="Incorrect unpacking"):
        A.create_acsr(m, 2, dev)


def test_headline_mask_on_device(dev):
    # L = 16384, window 512: rasterised and scanned on the GPU, checked against the closed form
    L, w = 16384, 512
    mask = A.create_causal_windowed_mask(L, w - 1, device=dev)
    got = A.create_acsr(mask, 16, dev)
    i = np.arange(L)
    a = np.maximum(0, i - w + 1).astype(np.float64)
    assert np.array_equal(bits(got[1]), bits(np.where(a == 0, 0.0, -a)))
    assert np.array_equal(bits(got[3]), bits(a))
    assert np.array_equal(bits(got[4]), bits(np.minimum(i + 1, w)))
    assert got[5] == w
    g = np.arange(L // 16)
    assert np.array_equal(bits(got[6]), bits(np.maximum(0, g * 16 - w + 1)))
    assert np.array_equal(bits(got[7]), bits(g * 16 + 16))


@pytest.mark.parametrize("kind,args,make", [
    ("blocked", (130, 7), lambda: O.create_blocked_mask(130, 7)),
    ("windowed", (100, 9), lambda: O.create_windowed_mask(100, 9)),
    ("causal", (256, 31), lambda: O.create_causal_windowed_mask(256, 31)),
    ("dilated", (200, 16, 3), lambda: O.create_dilated_mask(200, 16, 3)),
    ("strided", (300, 32, 16), lambda: O.create_strided_segment_masks(300, 32, 16))])
def test_mask_rasteriser(dev, kind, args, make):
    want = make()
    if kind == "blocked":
        got = [A.create_blocked_mask(*args, device=dev)]
    elif kind == "windowed":
        got = [A.create_windowed_mask(*args, device=dev)]
    elif kind == "causal":
        got = [A.create_causal_windowed_mask(*args, device=dev)]
    elif kind == "dilated":
        got = [A.dilated_pattern(*args).device_mask(dev)]
    else:
        got = [p.device_mask(dev) for p in A.strided_patterns(*args)]
    want = want if isinstance(want, list) else [want]
    for g, w in zip(got, want):
        assert g.dtype == torch.uint8 and np.array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("n,p,BH,BW", [(10, 2, 2, 2), (10, 2, 16, 16), (10, 2, 4, 16), (32, 10, 16, 16), (128, 57, 16, 16),
                                       (1024, 256, 16, 16)])
def test_preambles(dev, n, p, BH, BW):
    mask = A.create_blocked_mask(n, p)
    arr = np.asarray(mask)
    T = int(arr.sum(1).max())
    out, grid, tx, ty = r_sddmm.rsddmm_preamble(mask, (2, 2, n, T), BW, BH, dev, torch.bfloat16)
    xs, ys = O.naive_block_mappings(arr, BH, BW)
    assert tx.dtype == torch.int32 and np.array_equal(tx.cpu().numpy(), xs) and np.array_equal(ty.cpu().numpy(), ys)
    assert grid == O.rsddmm_grid(len(xs), (2, 2, n, T)) and tuple(out.shape) == (2, 2, n, T) and out.dtype == torch.bfloat16
    grid, out, full, pow2 = r_softmax.rsoftmax_preamble(mask, (2, 2, n, T), BW, dev, torch.float16)
    assert grid == O.rsoftmax_grid(n, BW, (2, 2, n, T)) and pow2 == O.rsoftmax_pow2(T) and full == (2, 2, n, T)
    out, grid, T2 = r_spmm.rspmm_preamble(mask, (2, 2, n, n), BW, BH, dev, torch.float32)
    assert T2 == T and grid == O.rspmm_grid((2, 2, n, n), BW, BH) and tuple(out.shape) == (2, 2, n, n)


def test_preamble_assertion(dev):
    with pytest.raises(AssertionError, match="Issues with generating arrangement"):
        r_sddmm.rsddmm_preamble(np.eye(4, dtype=np.uint8), (1, 1, 4, 1), 2, 1, dev, torch.float32)


def _pattern_cases():
    cases = []
    for s, p in [(1, 1), (10, 2), (130, 7), (128, 128), (100, 300), (1024, 328)]:
        cases.append(("blocked", A.blocked_pattern(s, p)))
    for s, p in [(1, 0), (64, 0), (100, 9), (333, 40), (50, 49), (50, 500)]:
        cases.append(("windowed", A.windowed_pattern(s, p)))
        cases.append(("causal", A.causal_windowed_pattern(s, p)))
    for s, w, dil in [(200, 16, 3), (300, 16, 3), (520, 64, 3), (2048, 512, 2), (64, 512, 2), (100, 1, 5), (77, 8, 1), (90, 7, 4)]:
        cases.append(("dilated", A.dilated_pattern(s, w, dil)))
    for s, loc, st in [(300, 32, 16), (1024, 128, 128), (100, 1, 1), (64, 200, 7), (257, 5, 300)]:
        for k, pat in enumerate(A.strided_patterns(s, loc, st)):
            cases.append((f"strided{k}", pat))
    return cases


@pytest.mark.parametrize("case", _pattern_cases(), ids=lambda c: f"{c[0]}-{c[1].s}-{c[1].p0}-{c[1].p1}")
@pytest.mark.parametrize("BH", [2, 16])
def test_closed_form_pattern_builder_equals_mask_scan(dev, case, BH):
    """splat_acsr_build_pattern (rows of the pattern in closed form, no mask) against splat_acsr_build on the
    rasterised pattern, which the tests above pin to the oracle: every output array bit for bit, T and the row-stride
    summary included; windows wider than the matrix, single-row matrices, dilations that run off either side."""
    pat = case[1]
    dev_t = torch.device(dev)
    a = A.build_acsr(pat, BH, dev_t)                       # closed form
    b = A.build_acsr(pat.device_mask(dev_t), BH, dev_t)    # scan of the rasterised mask
    for name in ("dTos_lin", "dTos_trans", "sTod_lin", "sTod_trans", "nnz", "span_start", "span_end"):
        assert np.array_equal(bits(getattr(a, name)), bits(getattr(b, name))), name
    assert torch.equal(a.row_first, b.row_first) and torch.equal(a.row_last, b.row_last)
    assert a.T == b.T and a.row_stride == b.row_stride


@pytest.mark.parametrize("case", _pattern_cases(), ids=lambda c: f"{c[0]}-{c[1].s}-{c[1].p0}-{c[1].p1}")
def test_transposed_patterns_in_closed_form(dev, case):
    """The transposed patterns (the backward pass plans its transposed products from their ACSR): the generator's
    transposed kind is the transpose of the rasterised pattern, and the closed-form builder on it equals the scan of
    that transpose, every output array bit for bit."""
    pat = case[1]
    dev_t = torch.device(dev)
    turned = pat.device_mask(dev_t).t().contiguous()
    assert torch.equal(pat.transposed().device_mask(dev_t), turned)
    assert pat.transposed().transposed() == pat
    a = A.build_acsr(pat.transposed(), 16, dev_t)
    b = A.build_acsr(turned, 16, dev_t)
    for name in ("dTos_lin", "dTos_trans", "sTod_lin", "sTod_trans", "nnz", "span_start", "span_end"):
        assert np.array_equal(bits(getattr(a, name)), bits(getattr(b, name))), name
    assert torch.equal(a.row_first, b.row_first) and torch.equal(a.row_last, b.row_last)
    assert a.T == b.T and a.row_stride == b.row_stride


def test_pattern_builder_needs_no_mask_for_long_sequences(dev):
    """L = 2^20 rows (a 1 TiB mask): metadata in closed form, checked against the per-pattern formulas."""
    L, w = 1 << 20, 512
    got = A.create_acsr(A.causal_windowed_pattern(L, w - 1), 16, dev)
    i = np.arange(L)
    a = np.maximum(0, i - w + 1).astype(np.float64)
    assert np.array_equal(bits(got[3]), bits(a)) and np.array_equal(bits(got[4]), bits(np.minimum(i + 1, w)))
    assert got[5] == w


def test_a_trailing_dimension_given_by_the_caller_spares_the_read_back(dev):
    """create_acsr(..., T=) returns the same arrays without reading the builder's record back; the record is read when
    a launcher first needs its hints, and a wrong figure is refused there."""
    import _splat_hip as hip
    L, p = 1024, 99
    pat = A.causal_windowed_pattern(L, p)
    A._MASK_CACHE.clear()
    got = A.create_acsr(pat, 16, dev, T=p + 1)
    assert A.build_acsr(pat, 16, dev).summary is not None        # nothing has been read back yet
    A._MASK_CACHE.clear()
    want = A.create_acsr(pat, 16, dev)
    assert got[5] == want[5] == p + 1
    for a, b in zip(got, want):
        if isinstance(a, torch.Tensor):
            assert torch.equal(a.view(torch.int32), b.view(torch.int32))
    assert int(got[3].splat_row_stride) == int(want[3].splat_row_stride) == 1 and int(got[3].splat_max_step) == 1
    # used by a launcher like any other metadata
    x = torch.rand(1, 1, L, p + 1, device=dev)
    y = torch.empty_like(x)
    r_softmax.rsoftmax_launcher(x, y, got[0], got[1], got[2], got[3], got[5], 128, got[4], (1, 1), 16)
    live = torch.arange(p + 1, device=dev)[None, :] < got[4][:, None]
    sums = torch.where(live, y[0, 0], torch.zeros((), device=dev)).sum(-1)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-5)
    # a wrong figure: refused when the metadata is first used (and at once when the build has been read back already)
    A._MASK_CACHE.clear()
    wrong = A.create_acsr(pat, 16, dev, T=p)
    z = torch.rand(1, 1, L, p, device=dev)
    with pytest.raises(hip.SplatError, match="longest row has 100"):
        r_softmax.rsoftmax_launcher(z, z, wrong[0], wrong[1], wrong[2], wrong[3], wrong[5], 128, wrong[4], (1, 1), 16)
    with pytest.raises(hip.SplatError, match="longest row has 100"):
        A.create_acsr(pat, 16, dev, T=p)
    A._MASK_CACHE.clear()
