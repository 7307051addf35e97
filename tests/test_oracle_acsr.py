"""Pins the oracle's ACSR builder (acsr_helpers.py:99-160 restated), the tile anchor maps
(r_sddmm.py:117-146) and the preamble bookkeeping against hand-derived known answers, per-pattern
closed forms, a slot->column round trip and numpy's own 2x2 solve."""
import numpy as np
import pytest

from oracle import splat_oracle as O

F = np.float32


def bits(x):
    return np.asarray(x, dtype=np.float32).view(np.uint32)


def assert_bits(got, want, what=""):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape, what
    assert np.array_equal(bits(got), bits(want)), f"{what}: {got} != {want}"


def test_known_answer_blocked_10_2():
    # create_blocked_mask(10, 2), BLOCK_HEIGHT=2, worked by hand:
    # rows 0-1 see {0,1}; rows 2-3 {0..3}; rows 4-5 {2..5}; rows 6-7 {4..7}; rows 8-9 {6..9}
    acsr = O.create_acsr(O.create_blocked_mask(10, 2), 2)
    assert_bits(acsr[0], [1] * 10, "dTos_lin")
    assert_bits(acsr[1], [0, 0, 0, 0, -2, -2, -4, -4, -6, -6], "dTos_trans")  # +0.0, not -0.0, for a = 0
    assert_bits(acsr[2], [1] * 10, "sTod_lin")
    assert_bits(acsr[3], [0, 0, 0, 0, 2, 2, 4, 4, 6, 6], "sTod_trans")
    assert_bits(acsr[4], [2, 2, 4, 4, 4, 4, 4, 4, 4, 4], "nnz")
    assert acsr[5] == 4
    assert_bits(acsr[6], [0, 0, 2, 4, 6], "span_start")
    assert_bits(acsr[7], [2, 4, 6, 8, 10], "span_end")
    assert all(a.dtype == np.float32 for a in acsr[:5] + acsr[6:])


def test_known_answer_irregular_rows():
    # row 0: ones at 3, 7, 8 -> anchors a=3, b=7 (only the first two count): solve [[3,1],[7,1]] x = [0,1]
    #        -> x = (1/4, -3/4); sparse->dense (4, 3/4); nnz 3; span end candidate 3*4 + 0.75
    # row 1: a single one at column 5 -> the (1, 0) branch, column lost by design
    # row 2: empty
    m = np.zeros((3, 10), np.uint8)
    m[0, [3, 7, 8]] = 1
    m[1, 5] = 1
    acsr = O.create_acsr(m, 2)
    assert_bits(acsr[0], [0.25, 1, 1])
    assert_bits(acsr[1], [-0.75, 0, 0])
    assert_bits(acsr[2], [4, 1, 1])
    assert_bits(acsr[3], [0.75, 0, 0])
    assert_bits(acsr[4], [3, 1, 0])
    assert acsr[5] == 3
    assert_bits(acsr[6], [0, 0])        # min(10, 0.75, 0) ; min(10, 0)
    assert_bits(acsr[7], [12.75, 0])    # max(-1, 12.75, 1) ; max(-1, 0)


def test_assertion_when_fewer_than_two_ones():
    m = np.zeros((2, 4), np.uint8)
    m[0, 1] = 2  # row sum 2 > 1 but no entry equals 1
    with pytest.raises(AssertionError, match="Incorrect unpacking"):
        O.create_acsr(m, 2)


@pytest.mark.parametrize("L,w,BH", [(64, 8, 16), (512, 64, 16), (100, 7, 16), (48, 48, 4), (33, 5, 2)])
def test_closed_form_causal_window(L, w, BH):
    acsr = O.create_acsr(O.create_causal_windowed_mask(L, w - 1), BH)
    i = np.arange(L)
    a = np.maximum(0, i - w + 1).astype(np.float64)
    assert_bits(acsr[0], np.ones(L))
    assert_bits(acsr[1], np.where(a == 0, 0.0, -a))
    assert_bits(acsr[2], np.ones(L))
    assert_bits(acsr[3], a)
    assert_bits(acsr[4], np.minimum(i + 1, w))
    assert acsr[5] == min(w, L)
    g = np.arange(-(-L // BH))
    assert_bits(acsr[6], np.maximum(0, g * BH - w + 1))
    assert_bits(acsr[7], np.minimum(g * BH + BH, L))  # nnz + a = i + 1 for the block's last row


@pytest.mark.parametrize("L,p", [(64, 3), (128, 16), (50, 60)])
def test_closed_form_window(L, p):
    acsr = O.create_acsr(O.create_windowed_mask(L, p), 16)
    i = np.arange(L)
    a = np.maximum(0, i - p).astype(np.float64)
    assert_bits(acsr[1], np.where(a == 0, 0.0, -a))
    assert_bits(acsr[3], a)
    assert_bits(acsr[4], np.minimum(i, p) + np.minimum(L - 1 - i, p) + 1)


@pytest.mark.parametrize("L,win,dil", [(64, 8, 2), (96, 16, 3), (256, 32, 2)])
def test_closed_form_dilated(L, win, dil):
    acsr = O.create_acsr(O.create_dilated_mask(L, win, dil), 16)
    i = np.arange(L)
    lo = i - (win * dil) // 2
    a = np.where(lo >= 0, lo, lo % dil).astype(np.float64)  # first column >= 0 congruent to lo
    t = np.arange(win)[None, :]
    cols = lo[:, None] + dil * t
    nnz = ((cols >= 0) & (cols < L)).sum(1)
    assert nnz.min() >= 2
    assert_bits(acsr[0], np.full(L, 1.0 / dil))
    assert_bits(acsr[1], np.where(a == 0, 0.0, -a / dil))
    assert_bits(acsr[2], np.full(L, dil))
    assert_bits(acsr[3], a / dil)
    assert_bits(acsr[4], nnz)


def test_closed_form_strided_far_segment():
    L, local, stride = 64, 8, 8
    _, far = O.create_strided_segment_masks(L, local, stride)
    acsr = O.create_acsr(far, 16)
    i = np.arange(L)
    # far columns: 7, 15, ... <= i - 8
    cnt = np.maximum(0, (i - local - (stride - 1)) // stride + 1)
    cnt = np.where(i - local >= stride - 1, cnt, 0)
    multi = cnt >= 2
    assert_bits(acsr[4], cnt)
    assert_bits(acsr[0], np.where(multi, 1.0 / stride, 1.0))
    assert_bits(acsr[1], np.where(multi, -(stride - 1) / stride, 0.0))
    assert_bits(acsr[2], np.where(multi, stride, 1))
    assert_bits(acsr[3], np.where(multi, (stride - 1) / stride, 0.0))


def test_solve_equals_closed_form_bitwise():
    # float32(np.linalg.solve([[a,1],[a+s,1]], [0,1])) == float32 of (1/s, -a/s) with +0.0 at a == 0
    for s in (1, 2, 3, 5, 7, 128):
        a = np.arange(0, 16385, dtype=np.int64)
        A = np.empty((a.size, 2, 2), np.int64)
        A[:, 0, 0], A[:, 0, 1], A[:, 1, 0], A[:, 1, 1] = a, 1, a + s, 1
        rhs = np.broadcast_to(np.array([0, 1], np.int64), (a.size, 2))[..., None]
        x = np.linalg.solve(A, rhs)[..., 0]
        x0 = np.full(a.size, 1.0 / s)
        x1 = np.where(a == 0, 0.0, -a.astype(np.float64) / s)
        assert np.array_equal(bits(x[:, 0].astype(F)), bits(x0.astype(F))), s
        assert np.array_equal(bits(x[:, 1].astype(F)), bits(x1.astype(F))), s
        assert np.array_equal(np.rint(1.0 / x[:, 0]).astype(np.int64), np.full(a.size, s))
        # span end: float32(nnz*s + |x1|) is insensitive to the last bits of the solve
        for nnz in (2, 63, 512):
            assert np.array_equal(bits((nnz * s + np.abs(x[:, 1])).astype(F)), bits((nnz * s + np.abs(x1)).astype(F)))


@pytest.mark.parametrize("make,BH", [
    (lambda: O.create_blocked_mask(32, 10), 16), (lambda: O.create_blocked_mask(16, 5), 2),
    (lambda: O.create_windowed_mask(40, 6), 16), (lambda: O.create_dilated_mask(48, 8, 3), 4),
    (lambda: O.create_strided_segment_masks(64, 8, 8)[1], 16)])
def test_vectorised_equals_rowwise(make, BH):
    m = make()
    v = O.instantiate_metadata(m, BH)
    r = O.instantiate_metadata_rowwise(m, BH)
    for key in ("dTos_lin", "dTos_trans", "sTod_lin", "sTod_trans", "nnz", "span_start", "span_end"):
        assert np.array_equal(np.asarray(v[key], np.float64), np.asarray(r[key], np.float64)), key


@pytest.mark.parametrize("make", [
    lambda: O.create_blocked_mask(128, 57), lambda: O.create_windowed_mask(64, 9),
    lambda: O.create_causal_windowed_mask(64, 15), lambda: O.create_dilated_mask(64, 8, 2),
    lambda: O.create_strided_segment_masks(96, 16, 16)[0]])
def test_slot_columns_round_trip(make):
    m = make()
    acsr = O.create_acsr(m, 16)
    cols, valid = O.slot_columns(acsr)
    for r in range(m.shape[0]):
        assert np.array_equal(cols[r][valid[r]], np.nonzero(m[r])[0]), r
        # dense -> sparse map sends those columns back to 0..nnz-1
        s = acsr[0][r].astype(np.float64) * cols[r][valid[r]] + acsr[1][r].astype(np.float64)
        assert np.allclose(s, np.arange(valid[r].sum()), atol=1e-3)


def test_single_column_rows_need_first_col():
    _, far = O.create_strided_segment_masks(64, 8, 8)
    acsr = O.create_acsr(far, 16)
    first, _ = O.row_extents(far)
    cols, valid = O.slot_columns(acsr, first_col=first)
    for r in range(64):
        assert np.array_equal(cols[r][valid[r]], np.nonzero(far[r])[0]), r


def test_tile_anchor_known_answers():
    m = O.create_blocked_mask(10, 2)
    xs, ys = O.naive_block_mappings(m, 2, 2)
    assert xs.tolist() == [0, 0, 2, 2, 4, 4, 6, 6, 8]
    assert ys.tolist() == [0, 2, 2, 4, 4, 6, 6, 8, 8]
    assert xs.dtype == np.int32 and ys.dtype == np.int32
    # one (partial) block when rows < BLOCK_HEIGHT
    xs, ys = O.naive_block_mappings(m, 16, 16)
    assert (xs.tolist(), ys.tolist()) == ([0], [0])
    # trailing partial row block is not visited: 10 rows, BH=4 -> blocks 0 and 1 only
    xs, ys = O.naive_block_mappings(m, 4, 16)
    assert ys.tolist() == [0, 4]
    # columns 0..4, BLOCK_WIDTH 2 -> anchors 0, 2 (4 is not < 4)
    m2 = np.zeros((2, 8), np.uint8)
    m2[:, :5] = 1
    assert O.naive_block_mappings(m2, 2, 2)[0].tolist() == [0, 2]
    with pytest.raises(AssertionError, match="Issues with generating arrangement"):
        O.naive_block_mappings(np.eye(4, dtype=np.uint8), 1, 2)


def test_preamble_bookkeeping():
    assert O.rsoftmax_pow2(4) == 4 and O.rsoftmax_pow2(5) == 8 and O.rsoftmax_pow2(191) == 256
    assert O.rsddmm_grid(9, (2, 3, 10, 4)) == (9, 6)
    assert O.rsoftmax_grid(10, 16, (2, 3, 10, 4)) == (1, 6)
    assert O.rspmm_grid((2, 3, 100, 64), 16, 16) == (4, 7, 6)
