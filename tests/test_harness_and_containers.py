"""The host containers of the ACSR (acsr_helpers.py:58-96 of the reference), the modules' own self-checks
(truth / is_correct / test of r_sddmm.py:186-256, r_softmax.py:152-224, r_spmm.py:166-261), the mask cache's keys and
the host-side argument checks that keep a launch from indexing past its metadata."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O
import acsr_helpers as A
import _splat_hip as hip
import r_sddmm
import r_softmax
import r_spmm
from r_attention import RegularAttention, attention_launcher

REF_SMALL = [(10, 2), (10, 5), (10, 7), (16, 5), (16, 16), (32, 10), (32, 20), (32, 32), (128, 57)]


def oracle_meta(mask, BH=16):
    t = O.create_acsr(np.asarray(mask), BH)
    return tuple(torch.from_numpy(x) if isinstance(x, np.ndarray) else x for x in t)


# ------------------------------------------------------------------ checkers, on the host (plain tensor code)
def test_is_correct_reads_the_first_column_attribute_before_it_slices():
    """Rows with one live column that is not column 0 (a strided far field's first rows): the metadata stores
    translation 0 for them (acsr_helpers.py:126-130), so the checkers need the builder's first-column array, which
    lives as an attribute on the translations tensor and would be lost by the checkers' own ``[:rows]`` slices."""
    far = O.create_strided_segment_masks(64, 8, 8)[1]          # row i: columns j <= i - 8 with j % 8 == 7
    counts = far.sum(1)
    assert (counts == 1).any() and far[counts == 1].argmax(1).min() > 0
    acsr_np = O.create_acsr(far, 16)
    first, _ = O.row_extents(far)
    meta = oracle_meta(far)
    meta[3].splat_first_col = torch.from_numpy(np.asarray(first)).int()
    g = torch.Generator().manual_seed(5)
    x = torch.randint(0, 100, (1, 2, 64, 64), generator=g).float()
    y = torch.randint(0, 100, (1, 2, 64, 64), generator=g).float()
    comp = O.sddmm(x, y, acsr_np, first_col=first)
    assert r_sddmm.is_correct(r_sddmm.truth(x, y, "cpu"), comp, meta[2], meta[3], meta[4], 1, 2, far.tolist())
    # without the attribute the single-column rows are looked up at column 0 and a correct result is rejected
    bare = oracle_meta(far)
    assert not r_sddmm.is_correct(r_sddmm.truth(x, y, "cpu"), comp, bare[2], bare[3], bare[4], 1, 2, far.tolist())
    p = torch.rand(1, 2, 64, int(acsr_np[5]), generator=g)
    out = O.spmm(p, y, acsr_np, first_col=first)
    assert r_spmm.is_correct(p, y, out, meta[2], meta[3], meta[4], 2, 1, far.tolist())
    assert not r_spmm.is_correct(p, y, out, bare[2], bare[3], bare[4], 2, 1, far.tolist())


@pytest.mark.parametrize("make", [lambda: O.create_blocked_mask(10, 2), lambda: O.create_blocked_mask(32, 10),
                                  lambda: O.create_causal_windowed_mask(40, 7), lambda: O.create_dilated_mask(48, 8, 2)])
def test_checkers_accept_the_oracle_and_reject_a_wrong_slot(make):
    mask = make()
    L = mask.shape[0]
    acsr_np = O.create_acsr(mask, 16)
    meta = oracle_meta(mask)
    g = torch.Generator().manual_seed(L)
    x = torch.randint(0, 100, (2, 2, L, L), generator=g).float()
    y = torch.randint(0, 100, (2, 2, L, L), generator=g).float()
    dense = r_sddmm.truth(x, y, "cpu")
    assert torch.equal(dense, O.truth(x, y))
    comp = O.sddmm(x, y, acsr_np)
    assert r_sddmm.is_correct(dense, comp, meta[2], meta[3], meta[4], 2, 2, mask.tolist())
    lv = torch.from_numpy(O.slot_columns(acsr_np)[1])
    r, s = [int(v[0]) for v in torch.nonzero(lv, as_tuple=True)]
    wrong = comp.clone()
    wrong[1, 0, r, s] += 0.5
    assert not r_sddmm.is_correct(dense, wrong, meta[2], meta[3], meta[4], 2, 2, mask.tolist())
    dead = comp.clone()
    dead[..., ~lv] = 1e9  # dead slots are not looked at
    assert r_sddmm.is_correct(dense, dead, meta[2], meta[3], meta[4], 2, 2, mask.tolist())

    probs = O.softmax_compressed(comp / 100.0, lv)
    assert r_softmax.is_correct(comp, probs, meta[2], meta[3], meta[4], 2, 2, mask.tolist())
    off = probs.clone()
    off[0, 1, r, s] += 0.02
    assert not r_softmax.is_correct(comp, off, meta[2], meta[3], meta[4], 2, 2, mask.tolist())

    p = torch.randint(0, 100, comp.shape, generator=g).float()
    v = torch.randint(0, 100, (2, 2, L, 24), generator=g).float()
    out = O.spmm(p, v, acsr_np)
    assert r_spmm.is_correct(p, v, out, meta[2], meta[3], meta[4], 2, 2, mask.tolist())
    bad = out.clone()
    bad[1, 1, r, 3] -= 1.0
    assert not r_spmm.is_correct(p, v, bad, meta[2], meta[3], meta[4], 2, 2, mask.tolist())


def test_live_slot_columns_follow_the_builders_rule():
    mask = O.create_dilated_mask(64, 8, 2)
    acsr_np = O.create_acsr(mask, 16)
    meta = oracle_meta(mask)
    cols, live = r_sddmm.live_slot_columns(meta[2], meta[3], meta[4], meta[5])
    want_cols, want_live = O.slot_columns(acsr_np)
    assert np.array_equal(live.numpy(), want_live)
    assert np.array_equal(cols.numpy()[want_live], want_cols[want_live])
    rr, ss = np.nonzero(want_live)
    assert np.all(mask[rr, cols.numpy()[rr, ss]] == 1)


def test_the_three_tests_keep_the_reference_assertion():
    for fn, args in ((r_sddmm.test, (8, 8, 9, 1, 1, None, 0, 16, 16, torch.float32)),
                     (r_softmax.test, (8, 9, 1, 1, None, 0, 16, torch.float32)),
                     (r_spmm.test, (8, 8, 9, 1, 1, None, 0, 16, 16, torch.float32))):
        with pytest.raises(AssertionError, match="We only need to consider the case when m=n."):
            fn(*args)


# ------------------------------------------------------------------ cache keys (no device needed)
def test_cache_keys_tell_views_and_edits_apart():
    m = torch.zeros(8, 8, dtype=torch.uint8)
    assert A._cache_key(m) != A._cache_key(m.t())           # same storage, other strides
    assert A._cache_key(m) != A._cache_key(m[1:])            # other storage offset and shape
    assert A._cache_key(m) != A._cache_key(m.view(torch.int8))
    k0 = A._cache_key(m)
    m[3, 3] = 1                                              # in-place edit bumps the version counter
    assert A._cache_key(m) != k0
    lst = [[0] * 6 for _ in range(6)]
    k1 = A._cache_key(lst)
    assert A._cache_key([row[:] for row in lst]) == k1       # equal contents, another object
    lst[2][4] = 1
    assert A._cache_key(lst) != k1                           # the same object, edited in place
    arr = np.zeros((6, 6), dtype=np.int64)
    k2 = A._cache_key(arr)
    arr[0, 0] = 1
    assert A._cache_key(arr) != k2
    assert A._cache_key(np.zeros((4, 9))) != A._cache_key(np.zeros((9, 4)))
    with pytest.raises(ValueError):
        A._cache_key([0, 1, 0])


# ------------------------------------------------------------------ on the device
@pytest.mark.gpu
@pytest.mark.parametrize("make,BH", [(lambda: O.create_blocked_mask(10, 2), 2), (lambda: O.create_dilated_mask(96, 16, 2), 16),
                                     (lambda: O.create_causal_windowed_mask(50, 6), 16)])
def test_instantiate_metadata_and_the_acsr_getters(dev, make, BH):
    """acsr_helpers.py:58-142: the containers hold what the oracle's instantiate_metadata computes, rounded to float32 as
    the device arrays store it."""
    mask = make()
    acsr = A.instantiate_metadata(mask.tolist(), BH, dev)
    assert isinstance(acsr, A.ACSR)
    assert all(isinstance(x, A.AffineIndices) for x in acsr.affine_indices)
    assert all(isinstance(x, A.AffineIndicesInt) for x in acsr.affine_indices_int)
    md = O.instantiate_metadata(mask, BH)
    f32 = lambda x: np.asarray(x, dtype=np.float64).astype(np.float32)
    bits = lambda x: np.asarray(x, dtype=np.float32).view(np.uint32)
    assert np.array_equal(bits(acsr.get_dTos_linear_transformations()), bits(f32(md["dTos_lin"])))
    assert np.array_equal(bits(acsr.get_dTos_translations()), bits(f32(md["dTos_trans"])))
    assert acsr.get_sTod_linear_transformations() == md["sTod_lin"].tolist()
    assert all(isinstance(x, int) for x in acsr.get_sTod_linear_transformations())
    assert np.array_equal(bits(acsr.get_sTod_translations()), bits(f32(md["sTod_trans"])))
    assert acsr.get_nnzs() == md["nnz"].tolist()
    spans = acsr.get_span_specialised_data()
    assert len(spans) == -(-mask.shape[0] // BH)
    assert np.array_equal(bits([s[0] for s in spans]), bits(f32(md["span_start"])))
    assert np.array_equal(bits([s[1] for s in spans]), bits(f32(md["span_end"])))
    if mask.shape[0] == 10:  # the hand-derived answer for the blocked 10/2 mask at block height 2
        assert acsr.get_nnzs() == [2, 2, 4, 4, 4, 4, 4, 4, 4, 4]
        assert acsr.get_dTos_translations() == [0, 0, 0, 0, -2, -2, -4, -4, -6, -6]
        assert acsr.get_sTod_translations() == [0, 0, 0, 0, 2, 2, 4, 4, 6, 6]
        assert spans == [(0, 2), (0, 4), (2, 6), (4, 8), (6, 10)]


@pytest.mark.gpu
def test_create_acsr_of_a_view_and_of_an_edited_mask(dev):
    m = torch.from_numpy(O.create_causal_windowed_mask(64, 5)).to(dev)
    a = A.create_acsr(m, 16, dev)
    at = A.create_acsr(m.t(), 16, dev)          # the transposed view shares storage, version and shape with m
    want_t = O.create_acsr(O.create_causal_windowed_mask(64, 5).T, 16)
    assert not torch.equal(a[3], at[3])
    for got, want in zip(at, want_t):
        if isinstance(want, np.ndarray):
            assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    lst = O.create_blocked_mask(32, 8).tolist()
    first = A.create_acsr(lst, 16, dev)
    lst[20][3] = 1                               # the same list object, edited in place
    second = A.create_acsr(lst, 16, dev)
    want = O.create_acsr(np.asarray(lst), 16)
    assert not torch.equal(first[3], second[3])
    for got, w in zip(second, want):
        if isinstance(w, np.ndarray):
            assert np.array_equal(got.cpu().numpy().view(np.uint32), w.view(np.uint32))
    # every call hands out tensors of its own
    again = A.create_acsr(lst, 16, dev)
    assert again[4].data_ptr() != second[4].data_ptr()
    again[4].zero_()
    assert torch.equal(A.create_acsr(lst, 16, dev)[4], second[4])


@pytest.mark.gpu
def test_metadata_of_another_mask_is_rejected_before_any_launch(dev):
    small = A.create_acsr_segments([A.causal_windowed_pattern(64, 7)], 16, dev)
    B, H, L, d = 1, 1, 128, 64
    q = torch.zeros(B, H, L, d, dtype=torch.float16, device=dev)
    with pytest.raises(hip.SplatError, match="entries"):
        attention_launcher(q, q.transpose(2, 3), q, torch.empty_like(q), small, 1.0)
    t = small.tuples[0]
    s_buf = torch.zeros(B, H, L, small.T, dtype=torch.float16, device=dev)
    with pytest.raises(hip.SplatError, match="entries"):
        r_sddmm.rsddmm_launcher(q, q.transpose(2, 3), s_buf, t[0], t[1], t[2], t[3], small.T, t[4], (1, 1), None, None, 16, 16)
    with pytest.raises(hip.SplatError, match="entries"):
        r_softmax.rsoftmax_launcher(s_buf, s_buf, t[0], t[1], t[2], t[3], small.T, 8, t[4], (1, 1), 16)
    with pytest.raises(hip.SplatError, match="entries"):
        r_spmm.rspmm_launcher(s_buf, q, torch.empty_like(q), t[0], t[1], t[2], t[3], t[6], t[7], small.T, t[4], (1, 1, 1), 16, 16)
    with pytest.raises(hip.SplatError, match="mask is"):
        RegularAttention(1, 128, 1, 64, A.causal_windowed_pattern(64, 7), 16, 16, dev, torch.float16)


@pytest.mark.gpu
def test_a_trailing_dimension_smaller_than_the_rows_counts_stays_inside_the_buffer(dev):
    """Metadata whose counts exceed the buffer's trailing dimension (a caller passing a smaller T than create_acsr
    returned): the kernels clamp every row to the slots the buffer has, so the guard rows after the buffer stay intact."""
    L, d, T_small = 128, 64, 8
    acsr = A.create_acsr(A.causal_windowed_pattern(L, 15), 16, dev)   # rows of up to 16 live columns
    assert acsr[5] == 16
    q, k, v = (t.to(dev) for t in O.make_inputs(3, 1, 1, L, d, torch.float16))
    SENT = 768.0
    buf = torch.full(((L + 4) * T_small,), SENT, dtype=torch.float16, device=dev)
    s_buf = buf[:L * T_small].view(1, 1, L, T_small)
    r_sddmm.rsddmm_launcher(q, k.transpose(2, 3), s_buf, acsr[0], acsr[1], acsr[2], acsr[3], T_small, acsr[4], (1, 1), None,
                            None, 16, 16, scale=0.125)
    r_softmax.rsoftmax_launcher(s_buf, s_buf, acsr[0], acsr[1], acsr[2], acsr[3], T_small, 8, acsr[4], (1, 1), 16)
    out = torch.empty(1, 1, L, d, dtype=torch.float16, device=dev)
    r_spmm.rspmm_launcher(s_buf, v, out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T_small, acsr[4], (1, 1, 1), 16, 16)
    torch.cuda.synchronize()
    assert torch.all(buf[L * T_small:] == SENT)
    assert torch.isfinite(out.float()).all()
    # each row attended over its first T_small live columns
    live = torch.arange(T_small, device=dev)[None, :] < acsr[4].clamp(max=T_small)[:, None]
    sums = torch.where(live, s_buf[0, 0].float(), torch.zeros((), device=dev)).sum(-1)
    assert torch.allclose(sums, torch.ones_like(sums), atol=1e-2)
    assert torch.all(s_buf[0, 0][~live] == SENT)


@pytest.mark.gpu
@pytest.mark.parametrize("n,p", REF_SMALL)
def test_the_modules_own_tests_pass_on_the_reference_cases(dev, n, p, capsys):
    """r_sddmm.py:258-410, r_softmax.py:226-386, r_spmm.py:263-441: B = H = 2, 16 x 16 blocks, blocked masks."""
    mask = A.create_blocked_mask(n, p)
    assert r_sddmm.test(n, n, n, 2, 2, mask, 0, 16, 16, torch.float32) is True
    assert r_softmax.test(n, n, 2, 2, mask, 0, 16, torch.float32) is True
    assert r_spmm.test(n, n, n, 2, 2, mask, 0, 16, 16, torch.float32) is True
    assert capsys.readouterr().out.count("test case passed!") == 3


@pytest.mark.gpu
def test_the_modules_own_tests_at_the_reference_large_case(dev):
    """The L = 1024 blocked cases the reference's author notes as failing (r_spmm.py:441)."""
    mask = A.create_blocked_mask(1024, 256)
    assert r_sddmm.test(1024, 64, 1024, 2, 2, mask, 0, 16, 16, torch.float32)
    assert r_softmax.test(1024, 1024, 2, 2, mask, 0, 16, torch.float32)
    assert r_spmm.test(1024, 1024, 1024, 2, 2, mask, 0, 16, 16, torch.float32)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n,p", REF_SMALL + [(1024, 256)])
def test_the_modules_own_tests_at_the_reference_dtype(dev, n, p, dtype, capsys):
    """The reference's ``__main__`` blocks call ``test`` with ``out_dtype=torch.bfloat16`` (r_sddmm.py:262-410,
    r_softmax.py:230-386, r_spmm.py:266-441).  What those calls print with the drop-in underneath:
      * SDDMM: passed -- inputs and ``truth`` are in the 16-bit type too, and both sides round the exact integer sum (fp32
        accumulation) to it the same way, so every live slot agrees bit for bit;
      * softmax: passed -- a row of 16-bit probabilities sums to 1 well within the rule's 1e-2;
      * SpMM: failed -- its inputs stay float32 and only the output is 16-bit, which cannot hold sums of products of
        integers below 100 to within 1e-3 (fp16 overflows to inf); the rule says so of any correct 16-bit result.
    The SpMM output is therefore also checked for what it should be: the exact sum, rounded once."""
    mask = A.create_blocked_mask(n, p)
    k = n if n < 1024 else 64
    assert r_sddmm.test(n, k, n, 2, 2, mask, 0, 16, 16, dtype) is True
    assert r_softmax.test(n, n, 2, 2, mask, 0, 16, dtype) is True
    assert r_spmm.test(n, n, n, 2, 2, mask, 0, 16, 16, dtype) is False
    out = capsys.readouterr().out
    assert out.count("test case passed!") == 2 and out.count("test case failed") == 1
    # the 16-bit SpMM output is the correctly rounded exact result
    acsr = A.create_acsr(mask, 16, dev)
    T = acsr[5]
    g = torch.Generator().manual_seed(n * 31 + p)
    left = torch.randint(0, 100, (2, 2, n, T), generator=g, dtype=torch.float32).to(dev)
    right = torch.randint(0, 100, (2, 2, n, n), generator=g, dtype=torch.float32).to(dev)
    got = torch.empty(2, 2, n, n, dtype=dtype, device=dev)
    r_spmm.rspmm_launcher(left, right, got, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4], (1, 1, 4), 16, 16)
    want = O.spmm(left.cpu().double(), right.cpu().double(), tuple(x.cpu().numpy() if isinstance(x, torch.Tensor) else x for x in acsr))
    assert torch.equal(got.cpu(), want.to(dtype))


def test_rows_that_are_not_arithmetic_progressions_are_found_on_the_host():
    """``non_affine_rows`` (the check behind the backward's refusal of masks whose transpose has no ACSR) on host tensors,
    with the metadata the oracle gives: the closed-form patterns and their transposes have none, a row with a stray
    column is named, and so is a row whose first, second and last column fit a progression that a middle column leaves."""
    for mask in (O.create_blocked_mask(40, 8), O.create_causal_windowed_mask(48, 9), O.create_dilated_mask(48, 8, 3),
                 sum(O.create_strided_segment_masks(64, 8, 8))[:, :], O.create_windowed_mask(33, 4)):
        for m in (mask, np.ascontiguousarray(mask.T)):
            if m is mask and m.shape[0] == 64:
                continue   # the union of the two strided segments is not one progression per row; its parts are
            acsr = O.create_acsr(m, 16)
            first, _ = O.row_extents(m)
            bad = A.non_affine_rows(torch.from_numpy(m.astype(np.uint8)), torch.from_numpy(np.asarray(first)),
                                    torch.from_numpy(acsr[2]), torch.from_numpy(acsr[4]))
            assert bad.numel() == 0
    m = O.create_causal_windowed_mask(48, 9).copy()
    m[30, 2] = 1                           # stray column in front of the window
    m[40] = 0
    m[40, [0, 2, 3, 6]] = 1                # first + step * (n - 1) = 6 is the last column, yet 3 is off the progression
    acsr = O.create_acsr(m, 16)
    first, _ = O.row_extents(m)
    bad = A.non_affine_rows(torch.from_numpy(m.astype(np.uint8)), torch.from_numpy(np.asarray(first)),
                            torch.from_numpy(acsr[2]), torch.from_numpy(acsr[4]))
    assert bad.tolist() == [30, 40]
