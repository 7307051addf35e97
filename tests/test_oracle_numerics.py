"""Cross-checks of the oracle's numeric operators: the compressed-layout pipeline (sddmm -> softmax ->
spmm) must reproduce textbook dense masked attention, and its pieces must satisfy the identities the
reference's own checkers test (row sums of 1, r_softmax.py:176; dot products over live slots, r_spmm.py:183-190)."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O


def _inputs(B, H, L, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, L, d, generator=g)
    k = torch.randn(B, H, L, d, generator=g)
    v = torch.randn(B, H, L, d, generator=g)
    return q, k.transpose(2, 3), v


MASKS = [lambda: O.create_blocked_mask(32, 10), lambda: O.create_causal_windowed_mask(48, 7),
         lambda: O.create_windowed_mask(40, 5), lambda: O.create_dilated_mask(64, 8, 2)]


@pytest.mark.parametrize("make", MASKS)
def test_pipeline_equals_dense_attention(make):
    m = make()
    L = m.shape[0]
    q, kT, v = _inputs(2, 2, L, 16)
    acsr = O.create_acsr(m, 16)
    s = O.sddmm(q, kT, acsr, scale=0.25)
    _, valid = O.slot_columns(acsr)
    p = O.softmax_compressed(s, torch.from_numpy(valid))
    out = O.spmm(p, v, acsr)
    ref = O.dense_masked_attention(q, kT, v, m, 0.25)
    assert torch.allclose(out, ref, atol=1e-5)
    # independent textbook evaluation with torch's own softmax
    mm = torch.from_numpy(m != 0)
    sc = (q @ kT * 0.25).masked_fill(~mm, float("-inf"))
    assert torch.allclose(ref, torch.softmax(sc, -1) @ v, atol=1e-5)
    # live slots sum to one
    live_sum = torch.where(torch.from_numpy(valid), p, torch.zeros(())).sum(-1)
    assert torch.allclose(live_sum, torch.ones_like(live_sum), atol=1e-5)


def test_sddmm_is_truth_at_slot_columns():
    m = O.create_blocked_mask(10, 2)
    q, kT, _ = _inputs(1, 1, 10, 10, seed=3)
    acsr = O.create_acsr(m, 16)
    s = O.sddmm(q, kT, acsr)
    dense = O.truth(q, kT)
    cols, valid = O.slot_columns(acsr)
    for r in range(10):
        for t in range(acsr[5]):
            if valid[r, t]:
                assert s[0, 0, r, t] == dense[0, 0, r, cols[r, t]]
            else:
                assert s[0, 0, r, t] == 0


def test_spmm_matches_explicit_dot_products():
    m = O.create_windowed_mask(12, 2)
    acsr = O.create_acsr(m, 16)
    g = torch.Generator().manual_seed(5)
    p = torch.rand(1, 1, 12, acsr[5], generator=g)
    v = torch.randn(1, 1, 12, 6, generator=g)
    out = O.spmm(p, v, acsr)
    cols, valid = O.slot_columns(acsr)
    for r in range(12):
        want = sum(p[0, 0, r, t] * v[0, 0, cols[r, t]] for t in range(acsr[5]) if valid[r, t])
        assert torch.allclose(out[0, 0, r], want, atol=1e-6)


def test_compress_decompress_round_trip():
    m = O.create_dilated_mask(32, 4, 2)
    acsr = O.create_acsr(m, 16)
    x = torch.randn(2, 1, 32, 32) * torch.from_numpy(m).float()
    assert torch.equal(O.decompress(O.compress(x, acsr), acsr, 32), x)


def test_empty_rows_give_zero_output():
    m = O.create_causal_windowed_mask(16, 3).copy()
    m[5] = 0
    q, kT, v = _inputs(1, 1, 16, 8)
    out = O.dense_masked_attention(q, kT, v, m, 1.0)
    assert torch.all(out[0, 0, 5] == 0) and torch.isfinite(out).all()


def test_chunked_equals_whole():
    m = O.create_causal_windowed_mask(64, 9)
    q, kT, v = _inputs(1, 2, 64, 16)
    whole = O.dense_masked_attention(q, kT, v, m, 0.3)
    chunked = O.dense_masked_attention_chunked(q, kT, v, lambda a, b: m[a:b] != 0, 0.3, row_chunk=24)
    assert torch.allclose(whole, chunked, atol=1e-6)


def test_two_segments_equal_union_mask():
    segs = O.create_strided_segment_masks(64, 8, 8)
    q, kT, v = _inputs(1, 1, 64, 16)
    union = segs[0] | segs[1]
    ref = O.dense_masked_attention(q, kT, v, union, 0.25)
    # per-segment compressed pipeline with a shared softmax
    acsrs = [O.create_acsr(s, 16) for s in segs]
    firsts = [O.row_extents(s)[0] for s in segs]
    sc = torch.cat([O.sddmm(q, kT, a, 0.25, first_col=f) for a, f in zip(acsrs, firsts)], -1)
    valid = np.concatenate([O.slot_columns(a)[1] for a in acsrs], -1)
    p = O.softmax_compressed(sc, torch.from_numpy(valid))
    T0 = acsrs[0][5]
    out = O.spmm(p[..., :T0], v, acsrs[0], first_col=firsts[0]) + O.spmm(p[..., T0:], v, acsrs[1], first_col=firsts[1])
    assert torch.allclose(out, ref, atol=1e-5)


def test_backward_reverse_mode_equals_closed_formulas_and_finite_differences():
    """The two statements of the gradients (autograd through the dense forward; dV = P^T dO, dS = P o (dP - rowsum)
    * scale, dQ = dS K, dK = dS^T Q) agree, and a central difference of the forward along a random direction matches
    their inner product with that direction."""
    L, d = 40, 8
    mask = O.create_windowed_mask(L, 5)
    mask[7] = 0  # an empty row: zero output, zero gradients through it
    g = torch.Generator().manual_seed(3)
    q, k, v, go = [torch.randn(1, 2, L, d, generator=g, dtype=torch.float64) for _ in range(4)]
    a = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, mask, 0.3, go)
    b = O.dense_masked_attention_grads_explicit(q, k.transpose(2, 3), v, mask, 0.3, go)
    for x, y in zip(a, b):
        assert float((x - y).abs().max()) <= 2e-5
    dq_, dk_, dv_ = [torch.randn(1, 2, L, d, generator=g, dtype=torch.float64) for _ in range(3)]
    f = lambda t: float((O.dense_masked_attention((q + t * dq_).float(), (k + t * dk_).float().transpose(2, 3),
                                                  (v + t * dv_).float(), mask, 0.3).double() * go).sum())
    h = 1e-2
    fd = (f(h) - f(-h)) / (2 * h)
    an = float((a[0].double() * dq_).sum() + (a[1].double() * dk_).sum() + (a[2].double() * dv_).sum())
    assert abs(fd - an) <= 2e-2 * max(1.0, abs(an))
    assert float(a[0][0, :, 7].abs().max()) == 0.0
