"""Fused forward and the three-kernel composition against fp32 dense masked attention (the oracle), at
the five benchmark configurations: small ones whole, large ones through a head subset plus size-independent
properties at full size."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O
import acsr_helpers as A
from r_attention import RegularAttention, attention_launcher, unit

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 2e-2}


def run_module(mask, B, H, L, d, dtype, dev, q, k, v, scale, fused, contig_kT=False):
    attn = RegularAttention(B, L, H, d, mask, 16, 16, dev, dtype, scale=scale, fused=fused)
    kT = k.to(dev).transpose(2, 3)
    if contig_kT:
        kT = kT.contiguous()
    out = attn([q.to(dev), kT, v.to(dev)])
    assert out is attn.rspmm_output
    return out.float().cpu()


def test_config1_fp32_whole(dev):
    """B=1, H=1, L=512, d=64, fp32, causal window 64, scale 1/sqrt(d)."""
    L, d = 512, 64
    mask = A.create_causal_windowed_mask(L, 63)  # list of lists, the reference's argument type
    q, k, v = O.make_inputs(1001, 1, 1, L, d, torch.float32)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, np.asarray(mask), d ** -0.5)
    for fused in (True, False):
        for contig in (False, True):
            got = run_module(mask, 1, 1, L, d, torch.float32, dev, q, k, v, d ** -0.5, fused, contig)
            assert float((got - want).abs().max()) <= TOL[torch.float32], (fused, contig)


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("contig", [False, True])
def test_config2_fp16(dev, fused, contig):
    """B=4, H=16, L=4096, d=64, fp16, causal window 256, inputs * 0.5: run whole on the GPU, checked on the
    first and last (batch, head) pairs."""
    B, H, L, d = 4, 16, 4096, 64
    q, k, v = O.make_inputs(1002, B, H, L, d, torch.float16, mul=0.5)
    mask = A.causal_windowed_pattern(L, 255)
    got = run_module(mask, B, H, L, d, torch.float16, dev, q, k, v, d ** -0.5, fused, contig)
    m = O.create_causal_windowed_mask(L, 255)
    for b, h in ((0, 0), (3, 15)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        want = O.dense_masked_attention_chunked(q[sl], k[sl].transpose(2, 3), v[sl], lambda a, c: m[a:c] != 0, d ** -0.5)
        assert float((got[sl] - want).abs().max()) <= TOL[torch.float16]


@pytest.mark.parametrize("fused", [True, False])
def test_config3_strided_two_segments(dev, fused):
    """B=2, H=16, L=8192, d=64, bf16, local 128 + every 128th column: two affine segments per row.  Run at
    H=2 (the per-head work is what scales), checked whole."""
    B, H, L, d = 1, 2, 8192, 64
    q, k, v = O.make_inputs(1003, B, H, L, d, torch.bfloat16)
    got = run_module(A.strided_patterns(L, 128, 128), B, H, L, d, torch.bfloat16, dev, q, k, v, d ** -0.5, fused)
    segs = O.create_strided_segment_masks(L, 128, 128)
    union = segs[0] | segs[1]
    want = O.dense_masked_attention_chunked(q, k.transpose(2, 3), v, lambda a, c: union[a:c] != 0, d ** -0.5)
    assert float((got - want).abs().max()) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("contig", [False, True])
def test_config4_dilated(dev, fused, contig):
    """B=2, H=32, L=8192, d=128, bf16, 512 keys centred on i with dilation 2.  Run at B=1, H=2."""
    B, H, L, d = 1, 2, 8192, 128
    q, k, v = O.make_inputs(1004, B, H, L, d, torch.bfloat16)
    got = run_module(A.dilated_pattern(L, 512, 2), B, H, L, d, torch.bfloat16, dev, q, k, v, d ** -0.5, fused, contig)
    m = O.create_dilated_mask(L, 512, 2)
    want = O.dense_masked_attention_chunked(q, k.transpose(2, 3), v, lambda a, c: m[a:c] != 0, d ** -0.5)
    assert float((got - want).abs().max()) <= TOL[torch.bfloat16]


@pytest.mark.parametrize("cfg", [3, 4])
def test_config3_and_config4_at_full_batch_and_heads(dev, cfg):
    """Configs 3 (B=2, H=16, L=8192, d=64, strided, two segments) and 4 (B=2, H=32, L=8192, d=128, dilated 512/2) at
    their full size, fused and unfused: the first and the last (batch, head) pair against the oracle, every pair through
    V = 1 gives 1."""
    if cfg == 3:
        B, H, L, d = 2, 16, 8192, 64
        pat = A.strided_patterns(L, 128, 128)
        segs = O.create_strided_segment_masks(L, 128, 128)
        dense = segs[0] | segs[1]
    else:
        B, H, L, d = 2, 32, 8192, 128
        pat = A.dilated_pattern(L, 512, 2)
        dense = O.create_dilated_mask(L, 512, 2)
    scale = d ** -0.5
    q, k, v = O.make_inputs(1000 + cfg, B, H, L, d, torch.bfloat16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    kT = kd.transpose(2, 3)
    wants = {}
    for b, h in ((0, 0), (B - 1, H - 1)):
        sl = (slice(b, b + 1), slice(h, h + 1))
        wants[(b, h)] = (sl, O.dense_masked_attention_chunked(q[sl], k[sl].transpose(2, 3), v[sl],
                                                              lambda a, c: dense[a:c] != 0, scale))
    for fused in (True, False):
        attn = RegularAttention(B, L, H, d, pat, 16, 16, dev, torch.bfloat16, scale=scale, fused=fused)
        got = attn([qd, kT, vd]).float().cpu()
        for sl, want in wants.values():
            assert float((got[sl] - want).abs().max()) <= TOL[torch.bfloat16], fused
        ones = attn([qd, kT, torch.ones_like(vd)]).float()
        assert float((ones - 1).abs().max()) <= TOL[torch.bfloat16], fused
        del attn


def test_config5_headline_full_size(dev):
    """B=4, H=16, L=16384, d=128, bf16, causal window 512, fused only: the full problem runs on the GPU;
    two (batch, head) pairs are checked against the oracle, the rest through properties that do not depend on
    size: V = 1 gives 1 (the weights of a row sum to one), and the output is linear in V."""
    B, H, L, d = 4, 16, 16384, 128
    scale = d ** -0.5
    q, k, v = O.make_inputs(1005, B, H, L, d, torch.bfloat16)
    attn = RegularAttention(B, L, H, d, A.causal_windowed_pattern(L, 511), 16, 16, dev, torch.bfloat16, scale=scale)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    for contig in (False, True):
        kT = kd.transpose(2, 3).contiguous() if contig else kd.transpose(2, 3)
        got = attn([qd, kT, vd]).float().cpu()
        m_rows = lambda a, c: ((np.arange(a, c)[:, None] >= np.arange(L)[None, :]) &
                               (np.arange(a, c)[:, None] - 511 <= np.arange(L)[None, :]))
        for b, h in ((0, 0), (3, 15)):
            sl = (slice(b, b + 1), slice(h, h + 1))
            want = O.dense_masked_attention_chunked(q[sl], k[sl].transpose(2, 3), v[sl], m_rows, scale)
            assert float((got[sl] - want).abs().max()) <= TOL[torch.bfloat16], (contig, b, h)
        assert torch.isfinite(got).all()
    kT = kd.transpose(2, 3)
    ones = attn([qd, kT, torch.ones_like(vd)]).float()
    assert float((ones - 1).abs().max()) <= 2e-2
    base = attn([qd, kT, vd]).float().clone()
    v2 = torch.randn(B, H, L, d, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).to(dev)
    o2 = attn([qd, kT, v2]).float().clone()
    o12 = attn([qd, kT, (vd.float() + v2.float()).to(torch.bfloat16)]).float()
    assert float((o12 - (base + o2)).abs().max()) <= 6e-2  # three bf16 roundings of O(1) values


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("make", [
    lambda: O.create_blocked_mask(128, 57), lambda: O.create_windowed_mask(333, 40),
    lambda: O.create_causal_windowed_mask(1000, 100), lambda: O.create_dilated_mask(520, 64, 3),
    lambda: O.create_blocked_mask(1024, 328)])
def test_fused_small_patterns(dev, dtype, d, make):
    mask = make()
    L = mask.shape[0]
    q, k, v = O.make_inputs(L + d, 2, 2, L, d, dtype)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, d ** -0.5)
    for contig in (False, True):  # K^T contiguous along the keys is the reference's layout, whatever L is
        got = run_module(mask, 2, 2, L, d, dtype, dev, q, k, v, d ** -0.5, True, contig)
        assert float((got - want).abs().max()) <= TOL[dtype], contig


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("L", [333, 1001])
def test_fused_reference_k_layout_with_ragged_length(dev, dtype, L):
    """The reference hands kT over as a contiguous [B, H, d, L] tensor (r_sddmm.py:230-231, r_attention.py:134-137).
    With L not a multiple of the 16-byte piece the key rows of that layout are not piece-aligned; the default (fused)
    forward must still take it."""
    d = 64
    mask = O.create_causal_windowed_mask(L, 77)
    q, k, v = O.make_inputs(7 * L, 1, 3, L, d, dtype)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, d ** -0.5)
    attn = RegularAttention(1, L, 3, d, mask, 16, 16, dev, dtype, scale=d ** -0.5)
    assert attn.fused
    kT = k.to(dev).transpose(2, 3).contiguous()
    assert kT.stride(3) == 1 and L % 8 != 0
    got = attn([q.to(dev), kT, v.to(dev)]).float().cpu()
    assert float((got - want).abs().max()) <= TOL[dtype]


def test_fused_views_that_are_not_piece_aligned(dev):
    """q, v and the output as views whose storage offset or row stride is not a multiple of 16 bytes: the launcher
    copies what the kernel cannot address piecewise and still writes the caller's output tensor."""
    B, H, L, d = 1, 2, 200, 64
    dtype = torch.float16
    mask = O.create_windowed_mask(L, 20)
    q, k, v = O.make_inputs(99, B, H, L, d, dtype)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, d ** -0.5)
    segs = A.create_acsr_segments([mask], 16, dev)

    def odd_view(t):  # same values, rows d + 3 elements apart, first element 3 elements into the storage
        buf = torch.zeros(B, H, L, d + 3, dtype=dtype, device=dev).flatten()
        buf = torch.cat([buf, buf.new_zeros(8)])
        view = buf[3:3 + B * H * L * (d + 3)].view(B, H, L, d + 3)[..., :d]
        view.copy_(t.to(dev))
        return view
    qv, vv, ov = odd_view(q), odd_view(v), odd_view(torch.zeros_like(q))
    assert qv.data_ptr() % 16 != 0 and qv.stride(2) % 8 != 0
    res = attention_launcher(qv, k.to(dev).transpose(2, 3), vv, ov, segs, d ** -0.5)
    assert res is ov
    assert float((ov.float().cpu() - want).abs().max()) <= TOL[dtype]


@pytest.mark.parametrize("name,make", [
    ("dilated, step 2", lambda: [A.dilated_pattern(640, 96, 2)]),
    ("strided far field", lambda: A.strided_patterns(768, 64, 32)),
    ("dense mask with stepping rows", lambda: [O.create_dilated_mask(300, 40, 3)]),
])
def test_gathered_rows_with_the_reference_layout_of_k(dev, name, make):
    """K^T stored contiguously along the keys (the reference's layout) and rows that step over columns: the launchers
    hand the kernels a row-major copy of K, so the results are those of row-major K bit for bit, for the fused forward
    and for rsddmm_launcher; a mask without stepping rows leaves the tensor as it is."""
    from r_sddmm import rsddmm_launcher
    pats = make()
    L = A.mask_shape(pats[0])[0]
    B, H, d, dtype = 2, 2, 64, torch.bfloat16
    q, k, v = [t.to(dev) for t in O.make_inputs(11, B, H, L, d, dtype)]
    segs = A.create_acsr_segments(pats, 16, dev)
    assert segs.gathered
    kT_rows, kT_cont = k.transpose(2, 3), k.transpose(2, 3).contiguous()
    assert segs.keys_as_rows(kT_cont).stride(2) == 1 and segs.keys_as_rows(kT_rows) is kT_rows
    outs = []
    for kT in (kT_rows, kT_cont):
        o = torch.empty(B, H, L, d, dtype=dtype, device=dev)
        attention_launcher(q, kT, v, o, segs, d ** -0.5)
        s = torch.full((B, H, L, segs.T), 3.0, dtype=dtype, device=dev)
        rsddmm_launcher(q, kT, s, None, None, None, None, segs.T, None, None, None, None, 16, 16, scale=d ** -0.5, segments=segs)
        outs.append((o, s))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])
    plain = A.create_acsr_segments([A.causal_windowed_pattern(L, 31)], 16, dev)
    assert not plain.gathered and plain.keys_as_rows(kT_cont) is kT_cont


def test_empty_and_single_column_rows(dev):
    L, d = 256, 64
    mask = O.create_causal_windowed_mask(L, 31).copy()
    mask[7] = 0          # empty row -> zero output
    mask[100] = 0
    mask[100, 40] = 1    # single live column that is not column 0
    q, k, v = O.make_inputs(5, 1, 2, L, d, torch.float16)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, 0.125)
    for fused in (True, False):
        got = run_module(mask, 1, 2, L, d, torch.float16, dev, q, k, v, 0.125, fused)
        assert float((got - want).abs().max()) <= TOL[torch.float16]
        assert torch.all(got[:, :, 7] == 0)


def test_unit_projection_wrapper(dev):
    """r_attention.py:102-110: project then attend (reference smoke test shape scaled down), default scale 1."""
    B, S, N, Hd = 2, 256, 4, 64
    g = torch.Generator().manual_seed(9)
    x = [torch.rand(B, S, N * Hd, generator=g) * 0.1 for _ in range(3)]
    w = [torch.rand(N * Hd, N, Hd, generator=g) * 0.1 for _ in range(3)]
    mask = A.create_windowed_mask(S, 32)
    attn = RegularAttention(B, S, N, Hd, mask, 16, 16, dev, torch.float32)
    got = unit(*[t.to(dev) for t in x], *[t.to(dev) for t in w], attn).cpu()
    q, k, v = [torch.einsum("bsd,dnh->bnsh", a, b) for a, b in zip(x, w)]
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, np.asarray(mask), 1.0)
    assert float((got - want).abs().max()) <= 1e-5


@pytest.mark.parametrize("L,d,w,dtype", [(32768, 128, 512, torch.bfloat16), (40003, 64, 300, torch.float16),
                                         (1 << 20, 128, 512, torch.bfloat16)])
def test_long_sequences_by_properties(dev, L, d, w, dtype):
    """Sequences longer than any benchmark configuration, one of them not a multiple of any tile size, one of a million
    rows: the mask never exists (`MaskPattern`: metadata in closed form), so the checks are size-independent ones:
    V = 1 gives 1 everywhere, and a few rows are recomputed directly from their window."""
    g = torch.Generator().manual_seed(L)
    q = torch.randn(1, 1, L, d, generator=g).to(dtype).to(dev)
    k = torch.randn(1, 1, L, d, generator=g).to(dtype).to(dev)
    v = torch.randn(1, 1, L, d, generator=g).to(dtype).to(dev)
    scale = d ** -0.5
    attn = RegularAttention(1, L, 1, d, A.causal_windowed_pattern(L, w - 1), 16, 16, dev, dtype, scale=scale)
    ones = attn([q, k.transpose(2, 3), torch.ones_like(v)]).float()
    assert float((ones - 1).abs().max()) <= TOL[dtype]
    out = attn([q, k.transpose(2, 3), v]).float()
    assert torch.isfinite(out).all()
    for r in (0, 1, w - 2, w - 1, w, L // 2 + 7, L - 2, L - 1):
        lo = max(0, r - w + 1)
        s = (q[0, 0, r].float() @ k[0, 0, lo:r + 1].float().T) * scale
        want = torch.softmax(s, -1) @ v[0, 0, lo:r + 1].float()
        assert float((out[0, 0, r] - want).abs().max()) <= TOL[dtype], r


def _random_affine_mask(rng, L):
    """Every row an arbitrary affine set a + step*t, t < cnt (what ACSR can represent), with empty rows,
    single-column rows and rows reaching the last column mixed in."""
    mask = np.zeros((L, L), dtype=np.uint8)
    for r in range(L):
        kind = rng.integers(0, 10)
        if kind == 0:
            continue  # empty row
        a = int(rng.integers(0, L))
        if kind == 1:
            mask[r, a] = 1  # single column
            continue
        step = int(rng.integers(1, max(2, L // 3)))
        cnt = int(rng.integers(2, max(3, (L - 1 - a) // step + 2)))
        cols = a + step * np.arange(cnt)
        cols = cols[cols < L]
        if kind == 2:  # run to the end of the row
            cols = np.arange(a, L, step)
        mask[r, cols] = 1
    return mask


@pytest.mark.parametrize("seed", range(6))
def test_random_affine_rows_against_oracle(dev, seed):
    """Rows with unrelated starts, steps and lengths (the dense-column plan, its per-position validity test, the
    first-column side channel of single-column rows), sizes that are no multiple of any tile, all three kernels'
    composition and the fused kernel, both 16-bit types and fp32."""
    rng = np.random.default_rng(1234 + seed)
    L = int(rng.integers(1, 330))
    d = (64, 128)[seed % 2]
    dtype = (torch.float32, torch.float16, torch.bfloat16)[seed % 3]
    mask = _random_affine_mask(rng, L)
    q, k, v = O.make_inputs(77 + seed, 1, 2, L, d, dtype)
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, d ** -0.5)
    for fused in (True, False):
        got = run_module(mask, 1, 2, L, d, dtype, dev, q, k, v, d ** -0.5, fused)
        assert float((got - want).abs().max()) <= TOL[dtype], (fused, L, d, dtype)
        assert torch.all(got[:, :, mask.sum(1) == 0] == 0)


def _plan_cases():
    rng = np.random.default_rng(99)
    return [
        ("causal window", lambda: A.causal_windowed_pattern(1000, 100), 1000, 64, torch.float16),
        ("two-sided window, ragged L", lambda: A.windowed_pattern(333, 40), 333, 128, torch.bfloat16),
        ("dilated (row-stride blocks)", lambda: A.dilated_pattern(1024, 128, 2), 1024, 128, torch.bfloat16),
        ("strided, two segments", lambda: A.strided_patterns(1024, 128, 128), 1024, 64, torch.bfloat16),
        ("blocked", lambda: O.create_blocked_mask(640, 128), 640, 64, torch.float32),
        ("random affine rows", lambda: _random_affine_mask(rng, 300), 300, 128, torch.float16),
    ]


@pytest.mark.parametrize("case", _plan_cases(), ids=lambda c: c[0])
def test_planned_forward_equals_unplanned(dev, case):
    """splat_attention_fwd derives every workgroup's tiles from the ACSR arrays, splat_attention_fwd_planned reads
    them from the plan built once per mask: the same kernel otherwise, so the outputs agree bit for bit, for row-major
    and key-contiguous K (the plan's two variants)."""
    _, make, L, d, dtype = case
    B, H = 2, 3
    attn = RegularAttention(B, L, H, d, make(), 16, 16, dev, dtype, scale=d ** -0.5)
    q, k, v = [t.to(dev) for t in O.make_inputs(L, B, H, L, d, dtype)]
    plan = A_plan(attn, L, dev)
    epc = 4 if dtype == torch.float32 else 8
    for contig in ((False, True) if L % epc == 0 else (False,)):
        kT = k.transpose(2, 3).contiguous() if contig else k.transpose(2, 3)
        a = torch.full((B, H, L, d), 7, dtype=dtype, device=dev)
        b = torch.full((B, H, L, d), 9, dtype=dtype, device=dev)
        attention_launcher(q, kT, v, a, attn.segments, attn.scale)
        attention_launcher(q, kT, v, b, attn.segments, attn.scale, plan)
        assert torch.equal(a, b), contig
        assert torch.equal(attn([q, kT, v]), a), contig  # the module plans by itself


def A_plan(attn, L, dev):
    from r_attention import attention_plan
    return attention_plan(attn.segments, L, dev)


def _masked_scores(q, k, mask, scale):
    s = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) * scale
    return s.masked_fill(torch.as_tensor(np.asarray(mask) == 0), float("-inf"))


@pytest.mark.parametrize("case", _plan_cases(), ids=lambda c: c[0])
def test_forward_with_stats(dev, case):
    """splat_attention_fwd_stats: the output is bit-identical to the other forwards' and lse equals torch.logsumexp
    of the masked, scaled fp32 scores (+inf on rows without live columns), with and without a plan."""
    name, make, L, d, dtype = case
    B, H = 2, 3
    mask = make()
    attn = RegularAttention(B, L, H, d, mask, 16, 16, dev, dtype, scale=d ** -0.5)
    q, k, v = O.make_inputs(5 * L, B, H, L, d, dtype)
    if isinstance(mask, np.ndarray):
        dense = mask
    else:
        # the device's rasterisation of a pattern is checked bit for bit against the oracle's masks elsewhere
        dense = sum(m.device_mask(dev).cpu().numpy() for m in (mask if isinstance(mask, list) else [mask]))
    want = torch.logsumexp(_masked_scores(q, k, dense, d ** -0.5), dim=-1)
    want = torch.where(torch.isinf(want), torch.full_like(want, float("inf")), want)   # empty rows: -inf -> +inf
    qd, kd, vd = [t.to(dev) for t in (q, k, v)]
    kT = kd.transpose(2, 3)
    plain = torch.empty_like(qd)
    attention_launcher(qd, kT, vd, plain, attn.segments, attn.scale)
    for plan in (None, A_plan(attn, L, dev)):
        out = torch.full_like(qd, 3)
        lse = torch.full((B, H, L), -7.0, device=dev)
        attention_launcher(qd, kT, vd, out, attn.segments, attn.scale, plan, lse)
        assert torch.equal(out, plain)
        got = lse.cpu()
        assert torch.equal(torch.isinf(got), torch.isinf(want))
        fin = torch.isfinite(want)
        assert float((got[fin] - want[fin]).abs().max()) <= 2e-5 * max(1.0, float(want[fin].abs().max())), name
    o2, l2 = attn.forward_with_stats([qd, kT, vd])
    assert torch.equal(o2, plain) and torch.equal(l2.cpu(), got)
    with pytest.raises(Exception, match="lse"):
        attention_launcher(qd, kT, vd, out, attn.segments, attn.scale, None, lse[:, :, :-1])


def test_partial_results_merge_through_lse(dev):
    """The two segments of the strided pattern run as two separate launches, merged row by row with their lse, give
    the two-segment launch's output and lse: what a caller that shards the keys does."""
    L, d, B, H = 2048, 128, 1, 2
    pats = A.strided_patterns(L, 128, 128)
    q, k, v = [t.to(dev) for t in O.make_inputs(321, B, H, L, d, torch.bfloat16)]
    kT = k.transpose(2, 3)
    outs, lses = [], []
    for m in ([pats[0]], [pats[1]], pats):
        attn = RegularAttention(B, L, H, d, m, 16, 16, dev, torch.bfloat16, scale=d ** -0.5)
        o, l = attn.forward_with_stats([q, kT, v])
        outs.append(o.float().clone())
        lses.append(l.clone())
    assert torch.isinf(lses[1][:, :, :128]).all() and torch.isfinite(lses[0]).all()   # no far columns before row 128
    tot = torch.logaddexp(lses[0], torch.where(torch.isinf(lses[1]), torch.full_like(lses[1], -float("inf")), lses[1]))
    w0 = torch.exp(lses[0] - tot).unsqueeze(-1)
    w1 = torch.where(torch.isinf(lses[1]), torch.zeros_like(tot), torch.exp(lses[1] - tot)).unsqueeze(-1)
    merged = w0 * outs[0] + w1 * outs[1]
    assert float((tot - lses[2]).abs().max()) <= 1e-4
    assert float((merged - outs[2]).abs().max()) <= TOL[torch.bfloat16]


def test_plan_arguments_are_checked(dev):
    import _splat_hip as hip
    L, d = 256, 64
    attn = RegularAttention(1, L, 1, d, A.causal_windowed_pattern(L, 31), 16, 16, dev, torch.float16)
    q = torch.zeros(1, 1, L, d, dtype=torch.float16, device=dev)
    plan = A_plan(attn, L, dev)
    with pytest.raises(hip.SplatError, match="bytes"):
        attention_launcher(q, q.transpose(2, 3), q, torch.empty_like(q), attn.segments, 1.0, plan[:-16])
    with pytest.raises(hip.SplatError):
        attention_launcher(q, q.transpose(2, 3), q, torch.empty_like(q), attn.segments, 1.0, plan.cpu())


@pytest.mark.parametrize("dtype,slope", [(torch.bfloat16, 0.5), (torch.float16, 0.125), (torch.float32, 0.5)])
def test_scores_that_outrun_the_first_tiles_reference(dev, dtype, slope):
    """Scores that grow along the keys: a row's later tiles exceed the maximum of its first tile by far more than the
    exponent range of the probabilities (e^96 for slope 0.5 over 192 keys; e^24 against fp16's 65504), so the kernel
    cannot keep the references its rows settled on and has to repeat the row block with moving references.  The same
    inputs with a short window never leave the fast path; both must match the oracle."""
    L, d = 512, 128
    q = torch.ones(1, 2, L, d)
    k = (slope * torch.arange(L, dtype=torch.float32) / d).view(1, 1, L, 1).expand(1, 2, L, d).contiguous()
    g = torch.Generator().manual_seed(11)
    v = torch.randn(1, 2, L, d, generator=g)
    q, k, v = [t.to(dtype) for t in (q, k, v)]
    for w in (255, 15):
        mask = O.create_causal_windowed_mask(L, w)
        want = O.dense_masked_attention(q, k.transpose(2, 3), v, mask, 1.0)
        got = run_module(mask, 1, 2, L, d, dtype, dev, q, k, v, 1.0, True)
        assert torch.isfinite(got).all(), w
        assert float((got - want).abs().max()) <= TOL[dtype], w


@pytest.mark.parametrize("dtype,d", [(torch.bfloat16, 128), (torch.float16, 64)])
def test_forward_and_backward_replay_from_a_captured_graph(dev, dtype, d):
    """The entry points neither allocate nor synchronise, so a caller may record them into a HIP graph: the fused forward
    (its plan built beforehand) and the fused backward are captured once and replayed on new inputs, with eager work and
    synchronisations between the replays, and every replay must equal the eager result on the same inputs."""
    from r_backward import attention_backward_fused
    B, H, L = 2, 2, 520
    scale = d ** -0.5
    attn = RegularAttention(B, L, H, d, A.causal_windowed_pattern(L, 150), 16, 16, dev, dtype, scale=scale)
    g = torch.Generator().manual_seed(11)
    q, k, v, go = [torch.randn(B, H, L, d, generator=g).to(dtype).to(dev) for _ in range(4)]
    x = [q, k.transpose(2, 3), v]
    out, lse = attn.forward_with_stats(x)                     # builds the plan and the statistics buffer
    attn.backward_pass(x, go, lse.clone(), out.clone())       # builds the transposed mask's ACSR and plan
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            o_g, lse_g = attn.forward_with_stats(x)
            grads_g = attention_backward_fused(q, x[1], v, o_g, go, lse_g, attn.segments, attn._segments_t, attn._plan,
                                               attn._plan_t, scale)
    torch.cuda.current_stream(dev).wait_stream(side)
    for seed in (1, 2, 3):
        gen = torch.Generator().manual_seed(seed)
        for t in (q, k, v, go):
            t.copy_(torch.randn(B, H, L, d, generator=gen).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        got_o, got_lse, got_g = o_g.clone(), lse_g.clone(), [t.clone() for t in grads_g]
        want_o, want_lse = attn.forward_with_stats(x)          # eager, same buffers as the captured forward writes
        want_o, want_lse = want_o.clone(), want_lse.clone()
        want_g = attn.backward_pass(x, go, want_lse, want_o)
        torch.cuda.synchronize()
        assert torch.equal(got_o, want_o) and torch.equal(got_lse, want_lse), seed
        for a, b_ in zip(got_g, want_g):
            assert torch.equal(a, b_), seed


def test_backward_with_listed_rows_replays_from_a_captured_graph(dev):
    """The same for a mask whose transposed far field is taken row by row (one more launch of the kernel and the kernel that
    adds the listed keys' shares, the schedule built by an eager call beforehand): every replay equals the eager result; and
    a capture that finds no schedule yet records the plain walk instead of building one."""
    from r_backward import attention_backward_fused, keys_side_schedule, transposed_segments
    B, H, L, d, dtype = 1, 2, 1100, 64, torch.bfloat16
    scale = d ** -0.5
    pats = A.strided_patterns(L, 48, 40)
    attn = RegularAttention(B, L, H, d, pats, 16, 16, dev, dtype, scale=scale)
    g = torch.Generator().manual_seed(12)
    q, k, v, go = [torch.randn(B, H, L, d, generator=g).to(dtype).to(dev) for _ in range(4)]
    x = [q, k.transpose(2, 3), v]
    out, lse = attn.forward_with_stats(x)
    attn.backward_pass(x, go, lse.clone(), out.clone(), sparse_rows=True)   # builds the transposed ACSR, the plans, the schedule
    assert keys_side_schedule(attn._segments_t, L, dev, B * H, always=True) is not None
    fresh_t = transposed_segments(pats, 16, dev)                             # no schedule attached to these yet
    fresh_plan_t = fresh_t.plan(L, dev)
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            o_g, lse_g = attn.forward_with_stats(x)
            grads_g = attention_backward_fused(q, x[1], v, o_g, go, lse_g, attn.segments, attn._segments_t, attn._plan,
                                               attn._plan_t, scale, sparse_rows=True)
            plain_g = attention_backward_fused(q, x[1], v, o_g, go, lse_g, attn.segments, fresh_t, attn._plan,
                                               fresh_plan_t, scale, sparse_rows=True)
    torch.cuda.current_stream(dev).wait_stream(side)
    assert not fresh_t.__dict__.get("_keys_side")                            # nothing was built under capture
    for seed in (1, 2, 3):
        gen = torch.Generator().manual_seed(seed)
        for t in (q, k, v, go):
            t.copy_(torch.randn(B, H, L, d, generator=gen).to(dtype))
        graph.replay()
        torch.cuda.synchronize()
        got_g, got_plain = [t.clone() for t in grads_g], [t.clone() for t in plain_g]
        want_o, want_lse = attn.forward_with_stats(x)
        want_o, want_lse = want_o.clone(), want_lse.clone()
        want_g = [t.clone() for t in attn.backward_pass(x, go, want_lse, want_o, sparse_rows=True)]
        want_plain = attn.backward_pass(x, go, want_lse, want_o, sparse_rows=False)
        torch.cuda.synchronize()
        for a, b_ in zip(got_g, want_g):
            assert torch.equal(a, b_), seed
        for a, b_ in zip(got_plain, want_plain):
            assert torch.equal(a, b_), seed
