"""Pins the oracle's mask generators (acsr_helpers.py:18-55 restated) with literal known answers and
closed-form row sums, then checks the product's list-of-lists generators against them."""
import numpy as np
import pytest

from oracle import splat_oracle as O
import acsr_helpers as A


def rows(*strings):
    return np.array([[int(c) for c in s] for s in strings], dtype=np.uint8)


def test_blocked_known_answer():
    # s=6, p=2: block 0 sees itself, block k sees blocks k-1 and k
    want = rows("110000", "110000", "111100", "111100", "001111", "001111")
    assert np.array_equal(O.create_blocked_mask(6, 2), want)
    # ragged: s=5, p=3 -> rows 3,4 are block 1 -> columns [0, 6) clipped to 5
    want = rows("11100", "11100", "11100", "11111", "11111")
    assert np.array_equal(O.create_blocked_mask(5, 3), want)


def test_windowed_known_answer():
    want = rows("11000", "11100", "01110", "00111", "00011")
    assert np.array_equal(O.create_windowed_mask(5, 1), want)
    assert np.array_equal(O.create_windowed_mask(3, 5), np.ones((3, 3), np.uint8))


def test_causal_windowed_known_answer():
    want = rows("10000", "11000", "11100", "01110", "00111")
    assert np.array_equal(O.create_causal_windowed_mask(5, 2), want)
    assert np.array_equal(O.create_causal_windowed_mask(4, 0), np.eye(4, dtype=np.uint8))


def test_dilated_known_answer():
    # window 2, dilation 2: columns i-2, i
    want = rows("100000", "010000", "101000", "010100", "001010", "000101")
    assert np.array_equal(O.create_dilated_mask(6, 2, 2), want)


def test_strided_known_answer():
    loc, far = O.create_strided_segment_masks(8, 2, 2)
    assert np.array_equal(loc, rows("10000000", "11000000", "01100000", "00110000", "00011000", "00001100", "00000110",
                                    "00000011"))
    # far: j <= i-2 and j odd
    assert np.array_equal(far, rows("00000000", "00000000", "00000000", "01000000", "01000000", "01010000", "01010000",
                                    "01010100"))
    assert not np.any(loc & far)


@pytest.mark.parametrize("s,p", [(10, 2), (10, 5), (10, 7), (16, 5), (16, 16), (32, 10), (128, 57), (97, 13)])
def test_row_sums_closed_form(s, p):
    i = np.arange(s)
    assert np.array_equal(O.create_windowed_mask(s, p).sum(1), np.minimum(i, p) + np.minimum(s - 1 - i, p) + 1)
    assert np.array_equal(O.create_causal_windowed_mask(s, p).sum(1), np.minimum(i, p) + 1)
    blk = O.create_blocked_mask(s, p)
    want = np.where(i < p, min(p, s), np.minimum((i // p + 1) * p, s) - (i // p - 1) * p)
    assert np.array_equal(blk.sum(1), want)
    w = O.create_windowed_mask(s, p)
    assert np.array_equal(w, w.T)
    assert np.array_equal(O.create_causal_windowed_mask(s, p), np.tril(w))


@pytest.mark.parametrize("s,p", [(10, 2), (10, 7), (16, 16), (32, 10), (33, 4), (7, 0)])
def test_product_generators_match(s, p):
    if p > 0:
        assert A.create_blocked_mask(s, p) == O.create_blocked_mask(s, p).tolist()
    assert A.create_windowed_mask(s, p) == O.create_windowed_mask(s, p).tolist()
    assert A.create_causal_windowed_mask(s, p) == O.create_causal_windowed_mask(s, p).tolist()
