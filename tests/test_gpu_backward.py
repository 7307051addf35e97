"""Backward pass (absent from the reference) against the oracle's dense gradients, and its own kernels against their
definitions on the compressed layout."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O
import acsr_helpers as A
from r_attention import RegularAttention, attention_with_grad
from r_backward import compressed_transpose_launcher, rspmm_t_launcher, softmax_backward_launcher, transposed_segments
from r_spmm import rspmm_launcher

pytestmark = pytest.mark.gpu

# Gradients pass through two 16-bit compressed matrices (probabilities and dS) before the last products: the bounds
# below are this build's own (the reference states none), about 4x what was measured on these inputs.
TOL = {torch.float32: 5e-5, torch.float16: 1.5e-2, torch.bfloat16: 8e-2}


def _cases():
    return [
        ("causal window", lambda: A.causal_windowed_pattern(300, 40), lambda: O.create_causal_windowed_mask(300, 40), 300),
        ("window", lambda: A.windowed_pattern(257, 33), lambda: O.create_windowed_mask(257, 33), 257),
        ("blocked", lambda: A.blocked_pattern(256, 64), lambda: O.create_blocked_mask(256, 64), 256),
        ("dilated", lambda: A.dilated_pattern(320, 32, 3), lambda: O.create_dilated_mask(320, 32, 3), 320),
        ("strided, two segments", lambda: A.strided_patterns(384, 32, 16),
         lambda: sum(O.create_strided_segment_masks(384, 32, 16)), 384),
    ]


@pytest.mark.parametrize("fused", [False, True], ids=["composed", "fused"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c[0])
def test_gradients_against_dense_attention(dev, case, dtype, fused):
    """Both backward passes (the operators composed over compressed matrices, and the fused kernel) against the oracle."""
    if fused and dtype == torch.float32:
        pytest.skip("the fused backward is built for 16-bit types; float32 takes the composed pass")
    _, make, dense, L = case
    B, H, d = 1, 2, 64
    scale = d ** -0.5
    q, k, v = O.make_inputs(L, B, H, L, d, dtype)
    go = O.make_inputs(L + 1, B, H, L, d, dtype)[0]
    want = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, np.asarray(dense()), scale, go)
    attn = RegularAttention(B, L, H, d, make(), 16, 16, dev, dtype, scale=scale)
    qd, kd, vd = [t.to(dev) for t in (q, k, v)]
    got = attn.backward_pass([qd, kd.transpose(2, 3), vd], go.to(dev), fused=fused)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], name
    # the same through autograd, K given as a contiguous [B, H, d, L] tensor underneath
    qa, ka, va = [t.clone().requires_grad_(True) for t in (qd, kd, vd)]
    out = attention_with_grad(qa, ka, va, attn)
    (out.float() * go.to(dev).float()).sum().backward()
    for name, g, w in zip(("dq", "dk", "dv"), (qa.grad, ka.grad, va.grad), want):
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], name


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", _cases(), ids=lambda c: c[0])
def test_probabilities_in_one_pass_and_gradients_with_the_forward_statistic(dev, case, dtype):
    """rsddmm_launcher(..., lse=) stores exp(scale * score - lse): with the statistic of the fused forward these are
    the probabilities that rsddmm + rsoftmax give (live slots equal within the type's rounding, dead slots untouched),
    and the backward pass that starts from them meets the oracle's gradients like the one that recomputes the softmax."""
    from r_sddmm import rsddmm_launcher
    from r_softmax import rsoftmax_launcher
    _, make, dense, L = case
    B, H, d = 2, 2, 64
    scale = d ** -0.5
    q, k, v = O.make_inputs(3 * L, B, H, L, d, dtype)
    go = O.make_inputs(3 * L + 1, B, H, L, d, dtype)[0]
    attn = RegularAttention(B, L, H, d, make(), 16, 16, dev, dtype, scale=scale)
    qd, kd, vd = [t.to(dev) for t in (q, k, v)]
    kT = kd.transpose(2, 3)
    _, lse = attn.forward_with_stats([qd, kT, vd])
    segs, T = attn.segments, attn.segments.T
    two = torch.full((B, H, L, T), 5, dtype=dtype, device=dev)
    rsddmm_launcher(qd, kT, two, None, None, None, None, T, None, None, None, None, 16, 16, scale=scale, segments=segs)
    rsoftmax_launcher(two, two, None, None, None, None, T, 0, None, None, 16, segments=segs)
    one = torch.full((B, H, L, T), 5, dtype=dtype, device=dev)
    rsddmm_launcher(qd, kT, one, None, None, None, None, T, None, None, None, None, 16, 16, scale=scale, segments=segs,
                    lse=lse)
    eps = {torch.float32: 2e-6, torch.float16: 2e-3, torch.bfloat16: 1.6e-2}[dtype]   # a few ulps of values <= 1
    assert float((one.float() - two.float()).abs().max()) <= eps
    assert torch.equal(one == 5, two == 5)   # the sentinel survives in exactly the same (dead) slots
    want = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, np.asarray(dense()), scale, go)
    got = attn.backward_pass([qd, kT, vd], go.to(dev), lse, fused=False)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], name
    with pytest.raises(Exception, match="lse"):
        rsddmm_launcher(qd, kT, one, None, None, None, None, T, None, None, None, None, 16, 16, scale=scale, segments=segs,
                        lse=lse[:, :1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("name,make,dense,L", [
    ("causal window over several row blocks and tiles", lambda: A.causal_windowed_pattern(700, 199), lambda: O.create_causal_windowed_mask(700, 199), 700),
    ("two-sided window", lambda: A.windowed_pattern(513, 130), lambda: O.create_windowed_mask(513, 130), 513),
    ("dilated, step 2", lambda: A.dilated_pattern(640, 96, 2), lambda: O.create_dilated_mask(640, 96, 2), 640),
    ("blocked", lambda: A.blocked_pattern(512, 128), lambda: O.create_blocked_mask(512, 128), 512),
    ("strided, two segments", lambda: A.strided_patterns(768, 64, 32), lambda: sum(O.create_strided_segment_masks(768, 64, 32)), 768),
], ids=lambda x: x if isinstance(x, str) else None)
def test_fused_backward(dev, name, make, dense, L, d, dtype):
    """The fused backward kernel at both head dimensions over masks that need several row blocks, several tiles per block,
    a last block that is not full and, for K, both memory layouts: against the oracle's dense gradients, and close to the
    composed pass on the same inputs."""
    B, H = 2, 2
    scale = d ** -0.5
    q, k, v = O.make_inputs(7 * L + d, B, H, L, d, dtype)
    go = O.make_inputs(7 * L + d + 1, B, H, L, d, dtype)[0]
    want = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, np.asarray(dense()), scale, go)
    attn = RegularAttention(B, L, H, d, make(), 16, 16, dev, dtype, scale=scale)
    qd, kd, vd, god = [t.to(dev) for t in (q, k, v, go)]
    out, lse = attn.forward_with_stats([qd, kd.transpose(2, 3), vd])
    got = attn.backward_pass([qd, kd.transpose(2, 3), vd], god, lse.clone(), out.clone(), fused=True)
    for nm, g, w in zip(("dq", "dk", "dv"), got, want):
        assert torch.isfinite(g.float()).all(), nm
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], nm
    # K^T stored contiguously (the reference's layout) and no forward results handed in: the forward that backward_pass
    # then runs walks dilated keys in another order, so its output and statistic may differ in their last bits
    got2 = attn.backward_pass([qd, kd.transpose(2, 3).contiguous(), vd], god, fused=True)
    for nm, a, b_ in zip(("dq", "dk", "dv"), got, got2):
        assert float((a.float() - b_.float()).abs().max().cpu()) <= TOL[dtype] / 4, nm
    composed = attn.backward_pass([qd, kd.transpose(2, 3), vd], god, lse, fused=False)
    for nm, a, b_ in zip(("dq", "dk", "dv"), got, composed):
        assert float((a.float() - b_.float()).abs().max().cpu()) <= 2 * TOL[dtype], nm


@pytest.mark.parametrize("d,dtype", [(64, torch.float16), (128, torch.bfloat16)])
def test_fused_backward_on_views_in_token_major_layout(dev, d, dtype):
    """q, k, v, the forward's output and the upstream gradient stored as [B, L, H, d] and handed over as [B, H, L, d]
    views (batch, head and row strides all differ from the contiguous ones; nothing is copied on the way in): the same
    bits as from contiguous tensors, on a mask with a ragged last block."""
    B, H, L = 2, 3, 333
    scale = d ** -0.5
    q, k, v = O.make_inputs(31 + d, B, H, L, d, dtype)
    go = O.make_inputs(32 + d, B, H, L, d, dtype)[0]
    attn = RegularAttention(B, L, H, d, A.windowed_pattern(L, 70), 16, 16, dev, dtype, scale=scale)
    cont = [t.to(dev) for t in (q, k, v, go)]

    def token_major(t):
        return t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    views = [token_major(t) for t in cont]
    assert all(t.stride(1) == d and t.stride(2) == H * d and not t.is_contiguous() for t in views)
    out_c, lse_c = attn.forward_with_stats([cont[0], cont[1].transpose(2, 3), cont[2]])
    out_c, lse_c = out_c.clone(), lse_c.clone()
    want = attn.backward_pass([cont[0], cont[1].transpose(2, 3), cont[2]], cont[3], lse_c, out_c, fused=True)
    want = [t.clone() for t in want]
    got = attn.backward_pass([views[0], views[1].transpose(2, 3), views[2]], views[3], lse_c, token_major(out_c), fused=True)
    for nm, a, b_ in zip(("dq", "dk", "dv"), got, want):
        assert torch.equal(a, b_), nm
    dense = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, np.asarray(O.create_windowed_mask(L, 70)), scale, go)
    for nm, g, w in zip(("dq", "dk", "dv"), got, dense):
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], nm


def _even_rows_far_field(L, local, stride):
    """Two segment masks: the causal window (i - local, i], and for even rows i the columns j <= i - local with
    j % stride == stride - 1.  The far segment's transpose keeps one key in ``stride``, whose queries step by 2."""
    i = np.arange(L)[:, None]
    j = np.arange(L)[None, :]
    near = ((j <= i) & (j > i - local)).astype(np.uint8)
    far = ((j <= i - local) & (j % stride == stride - 1) & (i % 2 == 0)).astype(np.uint8)
    return near, far


@pytest.mark.parametrize("name,make,dense,B,H,L,d,dtype", [
    ("strided 384/32/16", lambda: A.strided_patterns(384, 32, 16), lambda: sum(O.create_strided_segment_masks(384, 32, 16)),
     1, 2, 384, 64, torch.float16),
    ("strided 768/64/32, d = 128", lambda: A.strided_patterns(768, 64, 32), lambda: sum(O.create_strided_segment_masks(768, 64, 32)),
     2, 2, 768, 128, torch.bfloat16),
    ("strided 1000/48/40, ragged", lambda: A.strided_patterns(1000, 48, 40), lambda: sum(O.create_strided_segment_masks(1000, 48, 40)),
     1, 3, 1000, 64, torch.bfloat16),
    ("strided 3000/16/16: more than 128 listed keys", lambda: A.strided_patterns(3000, 16, 16),
     lambda: sum(O.create_strided_segment_masks(3000, 16, 16)), 1, 1, 3000, 64, torch.float16),
    ("far field of even rows only (columns step by 2), masks as arrays",
     lambda: [torch.from_numpy(m) for m in _even_rows_far_field(640, 32, 16)], lambda: sum(_even_rows_far_field(640, 32, 16)),
     1, 2, 640, 64, torch.float16),
], ids=lambda x: x if isinstance(x, str) else None)
def test_fused_backward_with_sparse_rows_of_the_transposed_mask_listed(dev, name, make, dense, B, H, L, d, dtype):
    """Segments of the transposed mask that keep few keys with long columns (a strided pattern's far field), taken row by
    row through splat_attention_bwd_keys: against the oracle's dense gradients, and within an ulp or two of the plain walk
    of 128 consecutive keys (a listed key's shares, one per stretch of queries, are rounded to the 16-bit type before they are added)."""
    from r_backward import keys_side_schedule
    scale = d ** -0.5
    q, k, v = O.make_inputs(11 * L + d, B, H, L, d, dtype)
    go = O.make_inputs(11 * L + d + 1, B, H, L, d, dtype)[0]
    want = O.dense_masked_attention_grads(q, k.transpose(2, 3), v, np.asarray(dense()), scale, go)
    attn = RegularAttention(B, L, H, d, make(), 16, 16, dev, dtype, scale=scale)
    qd, kd, vd, god = [t.to(dev) for t in (q, k, v, go)]
    x = [qd, kd.transpose(2, 3), vd]
    out, lse = attn.forward_with_stats(x)
    out, lse = out.clone(), lse.clone()
    listed = [t.clone() for t in attn.backward_pass(x, god, lse, out, fused=True, sparse_rows=True)]
    sched = keys_side_schedule(attn._segments_t, L, dev, B * H, always=True)
    assert sched is not None and len(sched.main) == 1 and sched.keys.numel() > 0
    plain = attn.backward_pass(x, god, lse, out, fused=True, sparse_rows=False)
    for nm, g, w, pl in zip(("dq", "dk", "dv"), listed, want, plain):
        assert torch.isfinite(g.float()).all(), nm
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], nm
        rel = (g.float() - pl.float()).abs() / pl.float().abs().clamp(min=1.0)
        assert float(rel.max()) <= 2 * torch.finfo(dtype).eps, nm
    assert torch.equal(listed[0], plain[0])   # dq does not depend on how the keys' side is walked


def test_keys_side_schedule_lists_every_entry_of_the_sparse_rows_once(dev):
    """The schedule's rows against the transposed segment they replace: per key, the stretches' progressions are disjoint
    and their union is the key's column of queries; padding rows are empty; masks without a row-sparse segment, and walks
    too short for the extra launch to pay, get no schedule."""
    from r_backward import keys_side_schedule
    L, local, stride = 2000, 48, 40
    segs_t = transposed_segments(A.strided_patterns(L, local, stride), 16, dev)
    assert keys_side_schedule(segs_t, L, dev, 4) is None            # columns of at most 31 tiles, one round: not worth it
    sched = keys_side_schedule(segs_t, L, dev, 4, always=True)
    assert sched is not None and len(sched.main) == 1 and sched.n_stretches > 1
    far_t = sum(O.create_strided_segment_masks(L, local, stride)[1:]).T     # [key, query]
    t = sched.rows.tuples[0]
    lin, nnz, fcol = t[2].cpu().numpy(), t[4].cpu().numpy().astype(np.int64), sched.rows.first_cols[0].cpu().numpy()
    key_of_row = sched.key_of_row.cpu().numpy()
    seen = np.zeros_like(far_t, dtype=np.int64)
    for r in range(sched.n_rows):
        if r % sched.per_stretch >= sched.keys.numel():
            assert nnz[r] == 0 and key_of_row[r] == -1
            continue
        assert key_of_row[r] == key_of_row[r % sched.per_stretch]     # the same keys in the same order in every stretch
        cols = fcol[r] + lin[r].astype(np.int64) * np.arange(nnz[r])
        seen[key_of_row[r], cols] += 1
    assert np.array_equal(seen, far_t.astype(np.int64))
    assert sorted(sched.keys.cpu().tolist()) == sorted(np.nonzero(far_t.sum(1))[0].tolist())
    # config 3's shape takes the schedule by itself; a causal window has nothing to list
    assert keys_side_schedule(transposed_segments(A.strided_patterns(8192, 128, 128), 16, dev), 8192, dev, 32) is not None
    assert keys_side_schedule(transposed_segments([A.causal_windowed_pattern(4096, 255)], 16, dev), 4096, dev, 64, always=True) is None


def test_fused_backward_at_config_3_by_comparison_of_the_two_walks(dev):
    """Config 3's full shape (bf16, B=2 H=16 L=8192 d=64, local window 128 + every 128th key): the default takes the far
    field's 63 keys row by row in 16 stretches of queries; same gradients as the plain walk within two ulps, and the
    keys nobody lists are bit-identical."""
    B, H, L, d, dtype = 2, 16, 8192, 64, torch.bfloat16
    scale = d ** -0.5
    attn = RegularAttention(B, L, H, d, A.strided_patterns(L, 128, 128), 16, 16, dev, dtype, scale=scale)
    g = torch.Generator(device=dev).manual_seed(3)
    q, k, v, go = (torch.randn(B, H, L, d, generator=g, device=dev).to(dtype) for _ in range(4))
    x = [q, k.transpose(2, 3), v]
    out, lse = attn.forward_with_stats(x)
    out, lse = out.clone(), lse.clone()
    got = [t.clone() for t in attn.backward_pass(x, go, lse, out, fused=True)]
    plain = attn.backward_pass(x, go, lse, out, fused=True, sparse_rows=False)
    from r_backward import keys_side_schedule
    sched = keys_side_schedule(attn._segments_t, L, dev, B * H)
    assert sched is not None and sched.keys.numel() == 63
    assert torch.equal(got[0], plain[0])
    listed = torch.zeros(L, dtype=torch.bool, device=dev)
    listed[sched.keys] = True
    for nm, a, b_ in zip(("dk", "dv"), got[1:], plain[1:]):
        assert torch.equal(a[:, :, ~listed], b_[:, :, ~listed]), nm
        diff = (a[:, :, listed].float() - b_[:, :, listed].float()).abs()
        assert float((diff / b_[:, :, listed].float().abs().clamp(min=1.0)).max()) <= 2 * torch.finfo(dtype).eps, nm


def test_keys_entry_point_checks_its_arguments(dev):
    import _splat_hip as hip
    L, d, B, H = 256, 64, 1, 1
    segs_t = transposed_segments(A.strided_patterns(L, 16, 16), 16, dev)
    from r_backward import keys_side_schedule
    sched = keys_side_schedule(segs_t, L, dev, B * H, always=True)
    R = sched.n_rows
    t = torch.zeros(B, H, L, d, device=dev, dtype=torch.float16)
    stat = torch.zeros(B, H, L, device=dev)
    part = torch.zeros(2, B, H, R, d, device=dev, dtype=torch.float16)
    plan = sched.rows.plan(R, dev)

    grads = torch.zeros(2, B, H, L, d, device=dev, dtype=torch.float16)

    def call(**kw):
        a = dict(q=t.data_ptr(), k=t.data_ptr(), keys=sched.key_of_row.data_ptr(), plan_bytes=plan.numel(), n_rows=R, d=d,
                 scale=0.125, sl=d, dk=grads[0].data_ptr(), dv=grads[1].data_ptr(), rps=sched.per_stretch)
        a.update(kw)
        rows = lambda ptr: [ptr, H * L * d, L * d, a["sl"]]
        return hip.lib().splat_attention_bwd_keys(*rows(a["q"]), *rows(a["k"]), *rows(t.data_ptr()), *rows(t.data_ptr()),
                                                  stat.data_ptr(), stat.data_ptr(), a["keys"], part[0].data_ptr(), part[1].data_ptr(),
                                                  sched.rows.seg_array(R), 1, plan.data_ptr(), a["plan_bytes"], B, H, L, a["n_rows"],
                                                  a["d"], a["scale"], hip.dtype_code(torch.float16), a["dk"], a["dv"], a["rps"],
                                                  hip.stream_ptr(dev))
    assert call() == 0
    assert call(dk=None, dv=None, rps=0) == 0      # the rows' shares only
    for kw, what in [(dict(q=None), "null"), (dict(keys=None), "null"), (dict(n_rows=0), "n_rows"), (dict(d=96), "head dim"),
                     (dict(scale=0.0), "scale"), (dict(plan_bytes=plan.numel() - 16), "plan"), (dict(q=t.data_ptr() + 2), "aligned"),
                     (dict(sl=d - 8), "row strides"), (dict(dv=None), "dk and dv"), (dict(rps=R - 1), "rows_per_stretch"),
                     (dict(rps=0), "rows_per_stretch"), (dict(dk=grads[0].data_ptr() + 2), "dk and dv")]:
        assert call(**kw) != 0, kw
        msg = hip.lib().splat_last_error().decode()
        assert what in msg, (kw, msg)
    torch.cuda.synchronize()


def test_fused_backward_arguments_are_checked(dev):
    from _splat_hip import SplatError
    L, d = 128, 64
    attn = RegularAttention(1, L, 1, d, A.causal_windowed_pattern(L, 15), 16, 16, dev, torch.float32, scale=0.125)
    q = torch.zeros(1, 1, L, d, device=dev)
    with pytest.raises(SplatError, match="16-bit"):
        attn.backward_pass([q, q.transpose(2, 3), q], q, fused=True)
    attn = RegularAttention(1, L, 1, d, A.causal_windowed_pattern(L, 15), 16, 16, dev, torch.bfloat16, scale=0.125)
    qb = q.to(torch.bfloat16)
    out, lse = attn.forward_with_stats([qb, qb.transpose(2, 3), qb])
    with pytest.raises(SplatError, match="lse"):
        attn.backward_pass([qb, qb.transpose(2, 3), qb], qb, lse[:, :, :-1], out, fused=True)
    with pytest.raises(SplatError, match="out"):
        attn.backward_pass([qb, qb.transpose(2, 3), qb], qb, lse, out[:, :, :-1], fused=True)


def test_softmax_backward_on_compressed_rows(dev):
    L = 200
    acsr = O.create_acsr(O.create_causal_windowed_mask(L, 30), 16)
    segs = A.create_acsr_segments([A.causal_windowed_pattern(L, 30)], 16, dev)
    T = segs.T
    g = torch.Generator().manual_seed(0)
    p = torch.rand(2, 3, L, T, generator=g)
    dp = torch.randn(2, 3, L, T, generator=g)
    valid = torch.from_numpy(O.slot_columns(acsr)[1])
    pm = torch.where(valid, p, torch.zeros_like(p))
    want = pm * (dp - (pm * dp).sum(-1, keepdim=True)) * 0.7
    ds = torch.full_like(p, 5.0).to(dev)
    softmax_backward_launcher(p.to(dev), dp.to(dev), ds, segs, 0.7)
    got = ds.cpu()
    assert float((got - want)[valid.expand_as(got)].abs().max()) <= 1e-5
    assert torch.all(got[~valid.expand_as(got)] == 5.0)  # dead slots untouched


@pytest.mark.parametrize("make,dense", [
    (lambda: [A.dilated_pattern(150, 16, 3)], lambda: [O.create_dilated_mask(150, 16, 3)]),
    (lambda: A.strided_patterns(200, 16, 8), lambda: O.create_strided_segment_masks(200, 16, 8))])
def test_compressed_transpose(dev, make, dense):
    masks, dms = make(), dense()
    L = dms[0].shape[0]
    segs = A.create_acsr_segments(masks, 16, dev)
    segs_t = transposed_segments(masks, 16, dev)
    g = torch.Generator().manual_seed(1)
    full = torch.randn(1, 2, L, L, generator=g)
    # (rows with a single live column keep that column only in the first-column side channel)
    src = torch.cat([O.compress(full, O.create_acsr(m, 16), first_col=O.row_extents(m)[0]) for m in dms], dim=-1)
    want = torch.cat([O.compress(full.transpose(2, 3).contiguous(), O.create_acsr(m.T.copy(), 16),
                                 first_col=O.row_extents(m.T.copy())[0]) for m in dms], dim=-1)
    dst = torch.zeros(1, 2, L, segs_t.T).to(dev)
    compressed_transpose_launcher(src.to(dev), dst, segs, segs_t)
    assert src.shape[-1] == segs.T and want.shape[-1] == segs_t.T
    assert torch.equal(dst.cpu(), want)


@pytest.mark.parametrize("dtype,n_out", [(torch.float32, 64), (torch.float32, 40), (torch.bfloat16, 128), (torch.float16, 24)])
@pytest.mark.parametrize("make,dense", [
    (lambda: [A.causal_windowed_pattern(300, 70)], lambda: [O.create_causal_windowed_mask(300, 70)]),
    (lambda: [A.blocked_pattern(256, 64)], lambda: [O.create_blocked_mask(256, 64)]),
    (lambda: [A.dilated_pattern(150, 16, 3)], lambda: [O.create_dilated_mask(150, 16, 3)]),
    (lambda: A.strided_patterns(200, 16, 8), lambda: O.create_strided_segment_masks(200, 16, 8))],
    ids=["causal window", "blocked", "dilated", "strided"])
def test_transposed_product(dev, make, dense, dtype, n_out):
    """out = (the compressed matrix as a dense one)^T . x, against that product in float64; and the same product from the
    stored transpose (splat_compressed_transpose + splat_spmm)."""
    masks, dms = make(), dense()
    L = dms[0].shape[0]
    segs = A.create_acsr_segments(masks, 16, dev)
    segs_t = transposed_segments(masks, 16, dev)
    g = torch.Generator().manual_seed(2)
    full = torch.randn(2, 2, L, L, generator=g).to(dtype)
    x = torch.randn(2, 2, L, n_out, generator=g).to(dtype)
    src = torch.cat([O.compress(full, O.create_acsr(m, 16), first_col=O.row_extents(m)[0]) for m in dms], dim=-1)
    live = torch.from_numpy(sum(np.asarray(m, dtype=np.int64) for m in dms) > 0)
    want = (torch.where(live, full.double(), torch.zeros((), dtype=torch.float64)).transpose(2, 3) @ x.double())
    out = torch.full((2, 2, L, n_out), 7.0, dtype=dtype).to(dev)
    rspmm_t_launcher(src.to(dev), x.to(dev), out, segs, segs_t)
    tol = {torch.float32: 2e-4, torch.float16: 6e-2, torch.bfloat16: 4e-1}[dtype]  # one rounding of sums of ~70 products
    assert float((out.double().cpu() - want).abs().max()) <= tol
    turned = torch.zeros(2, 2, L, segs_t.T, dtype=dtype).to(dev)
    compressed_transpose_launcher(src.to(dev), turned, segs, segs_t)
    out2 = torch.empty_like(out)
    rspmm_launcher(turned, x.to(dev), out2, None, None, None, None, None, None, segs_t.T, None, None, 16, 16, segments=segs_t)
    assert float((out.double() - out2.double()).abs().max().cpu()) <= tol


def _staircase_mask(L, seed, width):
    """Rows and columns both intervals of differing lengths (some empty): the lower and the upper column bound do not
    decrease from one row to the next."""
    rng = np.random.default_rng(seed)
    lo = np.sort(rng.integers(0, L, L))
    hi = np.maximum.accumulate(np.minimum(np.maximum(np.sort(rng.integers(0, L + width, L)), lo), lo + width))
    m = np.zeros((L, L), np.uint8)
    for r in range(L):
        m[r, lo[r]:min(hi[r], L)] = 1
    return m


MANY_BLOCKS_T = {
    # name: (segment masks, B*H, n_out, the plan table passed by hand)
    # the sequence fills neither the last block of columns nor the last tile of rows
    "causal127_L1000_n128": (lambda: [O.create_causal_windowed_mask(1000, 127)], 64, 128, False),
    "window63_L1000_n64": (lambda: [O.create_windowed_mask(1000, 63)], 64, 64, False),
    # blocks of columns grouped by a stride of 2 (a power of two) and of 3
    "dilated256x2_n128": (lambda: [O.create_dilated_mask(1024, 256, 2)], 64, 128, False),
    "dilated100x3_L1000_n64": (lambda: [O.create_dilated_mask(1000, 100, 3)], 64, 64, False),
    "blocked256_n128": (lambda: [O.create_blocked_mask(1024, 256)], 64, 128, False),
    # 26 tiles of rows per block of columns: more than the 16 whose row maps are prepared at a time
    "causal1500_L2048_n64": (lambda: [O.create_causal_windowed_mask(2048, 1500)], 32, 64, False),
    "staircase_n128": (lambda: [_staircase_mask(1024, 7, 300)], 64, 128, False),
    # rows of another column step than the blocks' (the far field): the launcher would pick the general kernel, so the table
    # is passed by hand; the kernel of thin wavefronts walks such rows a second time
    "strided32_16_two_segments_n64": (lambda: O.create_strided_segment_masks(1024, 32, 16), 64, 64, True),
}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", list(MANY_BLOCKS_T))
def test_transposed_product_16_bit_in_launches_of_many_blocks(dev, case, dtype):
    """16-bit transposed product with 64 / 128 output columns, here in launches of 512 blocks of 128 output rows: with the plan
    table of the transposed mask the kernel of thin wavefronts runs and must agree with the dense product and with the
    general kernel (plan=False); dead slots hold NaN and must not reach the output."""
    make, BH, n_out, by_hand = MANY_BLOCKS_T[case]
    dms = [np.asarray(m) for m in make()]
    L = dms[0].shape[0]
    segs = A.create_acsr_segments(dms, 16, dev)
    segs_t = transposed_segments(dms, 16, dev)
    g = torch.Generator(device=dev).manual_seed(61)
    full = torch.randn(1, BH, L, L, generator=g, device=dev).to(dtype)
    x = torch.randn(1, BH, L, n_out, generator=g, device=dev).to(dtype)
    src = torch.cat([O.compress(full, O.create_acsr(m, 16), first_col=O.row_extents(m)[0], fill=float("nan")) for m in dms], dim=-1)
    assert src.shape[-1] == segs.T
    live = torch.from_numpy(sum(m.astype(np.int64) for m in dms) > 0).to(dev)
    want = torch.where(live, full.float(), torch.zeros((), device=dev)).transpose(2, 3) @ x.float()
    del full
    # exact products of 16-bit values summed in float32: what is left is the output's own rounding (2^-9 / 2^-12 of a value)
    tol = {torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype] * float(want.abs().max())
    outs = []
    for plan in (segs_t.plan(L, dev) if by_hand else None, False):
        out = torch.full((1, BH, L, n_out), 7.0, dtype=dtype, device=dev)
        rspmm_t_launcher(src, x, out, segs, segs_t, plan=plan)
        assert torch.isfinite(out).all()
        assert float((out.float() - want).abs().max()) <= tol
        outs.append(out)
    assert segs_t.has_plan(L, dev)  # the first call built it (or the test did)
    assert float((outs[0].float() - outs[1].float()).abs().max()) <= tol


def test_transposed_product_at_config_4_by_column_sums_and_linearity(dev):
    """Config 4's full shape (B=2 H=32 L=8192, dilated 512/2, bf16, 128 features; 537 MB of probabilities): with x = 1 every
    feature of output row j is the sum of column j of the compressed matrix, which a scatter-add over the slots' columns
    gives without any dense matrix; and the product is linear in x."""
    B, H, L, d = 2, 32, 8192, 128
    pat = [A.dilated_pattern(L, 512, 2)]
    segs, segs_t = A.create_acsr_segments(pat, 16, dev), transposed_segments(pat, 16, dev)
    T = segs.T
    dm = O.create_dilated_mask(L, 512, 2)
    cols, valid = O.slot_columns(O.create_acsr(dm, 16), first_col=O.row_extents(dm)[0])
    lv = torch.from_numpy(valid).to(dev)
    ci = torch.from_numpy(np.where(valid, cols, 0)).to(dev)
    g = torch.Generator(device=dev).manual_seed(81)
    p = torch.rand(B, H, L, T, generator=g, device=dev)
    p = torch.where(lv, p, torch.full((), float("nan"), device=dev)).to(torch.bfloat16)
    want = torch.zeros(B * H, L, device=dev)
    want.scatter_add_(1, ci.reshape(1, -1).expand(B * H, -1), torch.nan_to_num(p.float()).reshape(B * H, -1))
    ones = torch.ones(B, H, L, d, device=dev, dtype=torch.bfloat16)
    out = torch.full((B, H, L, d), 7.0, dtype=torch.bfloat16, device=dev)
    rspmm_t_launcher(p, ones, out, segs, segs_t)
    assert segs_t.has_plan(L, dev)
    got = out.float().reshape(B * H, L, d)
    assert float((got - want[..., None]).abs().max()) <= 8e-3 * float(want.max())
    # linearity: (x1 + 2 x2) with values that bf16 adds exactly
    x1 = torch.randint(-4, 5, (B, H, L, d), generator=g, device=dev).to(torch.bfloat16)
    x2 = torch.randint(-4, 5, (B, H, L, d), generator=g, device=dev).to(torch.bfloat16)
    o1, o2, o3 = [torch.empty(B, H, L, d, dtype=torch.float32, device=dev) for _ in range(3)]
    # (float32 outputs take the general kernel: the two kernels against each other at full size)
    rspmm_t_launcher(p, x1, o1, segs, segs_t)
    rspmm_t_launcher(p, x2, o2, segs, segs_t)
    o3b = torch.empty(B, H, L, d, dtype=torch.bfloat16, device=dev)
    rspmm_t_launcher(p, x1 + 2 * x2, o3b, segs, segs_t)
    lin = o1 + 2 * o2
    assert float((o3b.float() - lin).abs().max()) <= 8e-3 * float(lin.abs().max())


def test_transposed_product_refuses_a_plan_that_is_too_small(dev):
    pat = [A.causal_windowed_pattern(1024, 100)]
    segs, segs_t = A.create_acsr_segments(pat, 16, dev), transposed_segments(pat, 16, dev)
    p = torch.zeros(8, 8, 1024, segs.T, device=dev, dtype=torch.bfloat16)
    x = torch.zeros(8, 8, 1024, 64, device=dev, dtype=torch.bfloat16)
    out = torch.zeros_like(x)
    plan = segs_t.plan(1024, dev)
    with pytest.raises(Exception, match="plan holds"):
        rspmm_t_launcher(p, x, out, segs, segs_t, plan=plan[:plan.numel() // 2])


def test_transposed_product_arguments_are_checked(dev):
    segs = A.create_acsr_segments([A.causal_windowed_pattern(64, 8)], 16, dev)
    segs_t = transposed_segments([A.causal_windowed_pattern(64, 8)], 16, dev)
    p = torch.zeros(1, 1, 64, segs.T, device=dev)
    x = torch.zeros(1, 1, 64, 32, device=dev)
    out = torch.zeros(1, 1, 64, 32, device=dev)
    from _splat_hip import SplatError
    with pytest.raises(SplatError):
        rspmm_t_launcher(p[..., :-1], x, out, segs, segs_t)
    with pytest.raises(SplatError):
        rspmm_t_launcher(p, x.transpose(2, 3), out, segs, segs_t)
    with pytest.raises(SplatError):
        rspmm_t_launcher(p, x[..., :16], out, segs, segs_t)


def test_backward_of_a_long_sequence_by_properties(dev):
    """L = 2^17 (no mask of that size exists anywhere: forward and transposed ACSR both come from the closed forms).
    With every row of V equal to one vector the output does not depend on q and k, so dq = dk = 0; with dO = 1 the
    columns of dV sum to the number of rows, because every row of the probabilities sums to 1."""
    L, d, w = 1 << 17, 64, 256
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, 1, L, d, generator=g).to(dtype).to(dev)
    k = torch.randn(1, 1, L, d, generator=g).to(dtype).to(dev)
    v0 = torch.randn(d, generator=g).to(dtype)
    v = v0.expand(1, 1, L, d).contiguous().to(dev)
    attn = RegularAttention(1, L, 1, d, A.causal_windowed_pattern(L, w - 1), 16, 16, dev, dtype, scale=d ** -0.5)
    go = torch.ones(1, 1, L, d, dtype=dtype, device=dev)
    dq, dk, dv = attn.backward_pass([q, k.transpose(2, 3), v], go)
    # dP~ is the same number in every slot of a row (exactly: the same dot product), so dS~ = P~ (dP~ - sum P~ dP~)
    # is rounding noise of the 16-bit probabilities
    assert float(dq.float().abs().max()) <= 0.05 and float(dk.float().abs().max()) <= 0.05
    col_sums = dv.float().sum(dim=2)  # [1, 1, d]
    assert float((col_sums / L - 1.0).abs().max()) <= 2e-3
    assert torch.isfinite(dv.float()).all()


def test_fused_backward_at_the_headline_shape_by_properties(dev):
    """The fused backward at the largest benchmark configuration (bf16, B=4, H=16, L=16384, d=128, causal window 512),
    where no dense reference fits: the pass is linear in the upstream gradient and scaling by 2 is exact in binary
    floating point, so doubling dO must double every gradient bit for bit; and the gradients of a few query rows (dq)
    and key rows (dk, dv) of one head are recomputed from their windows in fp32."""
    B, H, L, d, w = 4, 16, 16384, 128, 512
    dtype, scale = torch.bfloat16, 128 ** -0.5
    g = torch.Generator(device=dev).manual_seed(50)
    q, k, v, go = (torch.randn(B, H, L, d, generator=g, device=dev, dtype=torch.float32).to(dtype) for _ in range(4))
    attn = RegularAttention(B, L, H, d, A.causal_windowed_pattern(L, w - 1), 16, 16, dev, dtype, scale=scale)
    out, lse = attn.forward_with_stats([q, k.transpose(2, 3), v])
    out, lse = out.clone(), lse.clone()
    dq, dk, dv = [t.clone() for t in attn.backward_pass([q, k.transpose(2, 3), v], go, lse, out, fused=True)]
    dq2, dk2, dv2 = attn.backward_pass([q, k.transpose(2, 3), v], go * 2, lse, out, fused=True)
    for nm, a, b_ in (("dq", dq, dq2), ("dk", dk, dk2), ("dv", dv, dv2)):
        assert torch.isfinite(a.float()).all(), nm
        assert torch.equal(a * 2, b_), nm

    b, h = 3, 11
    qf, kf, vf, gf = (t[b, h].float() for t in (q, k, v, go))

    def rows_of_p(i0, i1):
        """P[i0:i1, :] restricted to the key range the rows can see, with that range's first key."""
        j0 = max(0, i0 - w + 1)
        s = (qf[i0:i1] @ kf[j0:i1].T) * scale
        ii = torch.arange(i0, i1, device=dev)[:, None]
        jj = torch.arange(j0, i1, device=dev)[None, :]
        s = torch.where((jj <= ii) & (jj > ii - w), s, torch.full_like(s, float("-inf")))
        return torch.softmax(s, dim=-1), j0

    def ds_of(i0, i1):
        p, j0 = rows_of_p(i0, i1)
        dp = gf[i0:i1] @ vf[j0:i1].T
        return p, p * (dp - (p * dp).sum(-1, keepdim=True)) * scale, j0

    tol = TOL[dtype]
    for i0 in (0, 700, 8191, L - 64):      # 64 query rows each
        p, ds, j0 = ds_of(i0, i0 + 64)
        assert float((dq[b, h, i0:i0 + 64].float() - ds @ kf[j0:i0 + 64]).abs().max()) <= tol, i0
    for j in (0, 300, 9000, L - 3):        # one key row each: its queries are j .. j + w - 1
        i1 = min(L, j + w)
        p, ds, j0 = ds_of(j, i1)
        assert float((dk[b, h, j].float() - ds[:, j - j0] @ qf[j:i1]).abs().max()) <= tol, j
        assert float((dv[b, h, j].float() - p[:, j - j0] @ gf[j:i1]).abs().max()) <= tol, j


def _dead_ends_mask(L=256, p=31):
    """Causal window with the last row emptied (so the last key column is seen by no query) and the row before it cut
    down to its diagonal entry (a single live column that is not column 0).  Both cuts take the last entries of the
    columns they touch, so every column still meets an arithmetic progression of rows."""
    mask = O.create_causal_windowed_mask(L, p).copy()
    mask[L - 1] = 0
    mask[L - 2, :L - 2] = 0
    return mask


@pytest.mark.parametrize("fused", [False, True], ids=["composed", "fused"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gradients_with_an_empty_row_a_single_column_row_and_an_unseen_key(dev, dtype, fused):
    """The forward gives an empty row out = 0 and lse = +inf; the backward recomputes exp(score - lse) from that and
    must come out with zeros there, not NaN: the empty query row's dq, and dk / dv of the key nobody attends to."""
    L, d, B, H = 256, 64, 1, 2
    mask = _dead_ends_mask(L)
    scale = d ** -0.5
    q, k, v = O.make_inputs(77, B, H, L, d, dtype)
    go = O.make_inputs(78, B, H, L, d, dtype)[0]
    want = O.dense_masked_attention_grads_explicit(q, k.transpose(2, 3), v, mask, scale, go)
    attn = RegularAttention(B, L, H, d, torch.from_numpy(mask), 16, 16, dev, dtype, scale=scale)
    qd, kd, vd = [t.to(dev) for t in (q, k, v)]
    got = attn.backward_pass([qd, kd.transpose(2, 3), vd], go.to(dev), fused=fused)
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert torch.isfinite(g.float()).all(), name
        assert float((g.float().cpu() - w).abs().max()) <= TOL[dtype], name
    dq, dk, dv = got
    assert torch.all(dq[:, :, L - 1] == 0)
    assert torch.all(dk[:, :, L - 1] == 0) and torch.all(dv[:, :, L - 1] == 0)


def test_a_mask_whose_columns_are_not_affine_is_refused_by_the_backward(dev):
    """Rows affine, columns not: the forward runs, the backward raises instead of handing out wrong dk / dv."""
    from _splat_hip import SplatError
    L, d = 256, 64
    mask = O.create_causal_windowed_mask(L, 31).copy()
    mask[100] = 0
    mask[100, 40] = 1                      # column 40 now meets rows 40..71 and 100
    attn = RegularAttention(1, L, 1, d, torch.from_numpy(mask), 16, 16, dev, torch.float16, scale=0.125)
    q, k, v = [t.to(dev) for t in O.make_inputs(5, 1, 1, L, d, torch.float16)]
    out = attn([q, k.transpose(2, 3), v]).float().cpu()
    want = O.dense_masked_attention(q.cpu(), k.cpu().transpose(2, 3), v.cpu(), mask, 0.125)
    assert float((out - want).abs().max()) <= 1e-2
    with pytest.raises(SplatError, match="arithmetic progression"):
        attn.backward_pass([q, k.transpose(2, 3), v], torch.ones_like(q))
    with pytest.raises(SplatError, match="column 40"):
        transposed_segments([torch.from_numpy(mask)], 16, dev)
    # the same rows without the stray entry: accepted
    ok = O.create_causal_windowed_mask(L, 31)
    assert len(transposed_segments([torch.from_numpy(ok)], 16, dev)) == 1
