"""SDDMM, softmax and SpMM HIP kernels against the oracle on identical seeded inputs."""
import numpy as np
import pytest
import torch

from oracle import splat_oracle as O
import acsr_helpers as A
import r_sddmm
import r_softmax
import r_spmm

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.float16: 1e-2, torch.bfloat16: 2e-2}
SENTINEL = 768.0  # exactly representable in bf16 and fp16


def acsr_pair(mask, BH, dev):
    return A.create_acsr(mask, BH, dev), O.create_acsr(np.asarray(mask), BH)


def live(acsr_np):
    return torch.from_numpy(O.slot_columns(acsr_np)[1])


REF_SMALL = [(10, 2), (10, 5), (10, 7), (16, 5), (16, 16), (32, 10), (32, 20), (32, 32), (128, 57)]


# ---------------------------------------------------------------- SDDMM
@pytest.mark.parametrize("n,p", REF_SMALL)
def test_sddmm_reference_cases(dev, n, p):
    """r_sddmm.py:224-256 with its masks: m = k = n, B = H = 2, 16x16 blocks, integer-valued inputs, the
    reference's acceptance rule |out[r, s] - truth[r, c(r, s)]| <= 1e-3 on live slots (exact here: integer
    products below 2^24 summed in fp32)."""
    mask = A.create_blocked_mask(n, p)
    g = torch.Generator().manual_seed(n * 100 + p)
    left = torch.randint(0, 100, (2, 2, n, n), generator=g).float()
    right = torch.randint(0, 100, (2, 2, n, n), generator=g).float()
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    out, grid, tx, ty = r_sddmm.rsddmm_preamble(mask, (2, 2, n, acsr[5]), 16, 16, dev, torch.float32)
    out.fill_(SENTINEL)
    res = r_sddmm.rsddmm_launcher(left.to(dev), right.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[5], acsr[4],
                                  grid, tx, ty, 16, 16)
    assert res[0] is out and res[1] is acsr[2] and res[2] is acsr[3] and res[3] is acsr[4]
    want = O.sddmm(left, right, acsr_np)
    lv = live(acsr_np)
    got = out.cpu()
    assert torch.all(torch.abs(got - want)[..., lv] <= 1e-3)
    assert torch.all(got[..., ~lv] == SENTINEL), "dead slots must not be written"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["view", "contig"])
@pytest.mark.parametrize("make,d", [
    (lambda: O.create_causal_windowed_mask(512, 63), 64), (lambda: O.create_windowed_mask(300, 20), 40),
    (lambda: O.create_dilated_mask(256, 32, 2), 128), (lambda: O.create_blocked_mask(200, 33), 200),
    (lambda: O.create_causal_windowed_mask(130, 9), 10)])
def test_sddmm_patterns(dev, dtype, layout, make, d):
    mask = make()
    L = mask.shape[0]
    q, k, _ = O.make_inputs(11, 2, 3, L, d, dtype)
    kT = k.transpose(2, 3)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    scale = d ** -0.5
    want = O.sddmm(q, kT, acsr_np, scale)
    kT_dev = k.to(dev).transpose(2, 3)
    if layout == "contig":
        kT_dev = kT_dev.contiguous()
    out = torch.full((2, 3, L, acsr[5]), SENTINEL, dtype=dtype, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), kT_dev, out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[5], acsr[4], (1, 1),
                            None, None, 16, 16, scale=scale)
    got = out.float().cpu()
    lv = live(acsr_np)
    tol = TOL[dtype] * max(1.0, float(want.abs().max()))
    assert float((got - want)[..., lv].abs().max()) <= tol
    assert torch.all(got[..., ~lv] == SENTINEL)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["view", "contig"])
@pytest.mark.parametrize("make,d", [
    (lambda: O.create_causal_windowed_mask(1024, 511), 64),   # whole-line output path of the 16-bit types
    (lambda: O.create_windowed_mask(300, 20), 40), (lambda: O.create_dilated_mask(256, 32, 2), 128),
    (lambda: O.create_blocked_mask(200, 33), 200), (lambda: O.create_causal_windowed_mask(130, 9), 10)])
def test_sddmm_probabilities_from_a_row_statistic(dev, dtype, layout, make, d):
    """rsddmm_launcher(..., lse=): exp(scale * score - lse[row]) in the live slots, nothing in the dead ones; with
    lse = torch.logsumexp of the row's live scaled scores that is the oracle's compressed softmax of its SDDMM.  Head
    widths the fused kernel does not take, contractions longer than one staging chunk, both K layouts."""
    mask = make()
    L = mask.shape[0]
    q, k, _ = O.make_inputs(13, 2, 3, L, d, dtype)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    scale = d ** -0.5
    scores = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) * scale
    lse = torch.logsumexp(scores.masked_fill(torch.as_tensor(mask == 0), float("-inf")), dim=-1)
    want = O.softmax_compressed(O.sddmm(q, k.transpose(2, 3), acsr_np, scale), live(acsr_np))
    kT_dev = k.to(dev).transpose(2, 3)
    if layout == "contig":
        kT_dev = kT_dev.contiguous()
    out = torch.full((2, 3, L, acsr[5]), SENTINEL, dtype=dtype, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), kT_dev, out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[5], acsr[4], (1, 1),
                            None, None, 16, 16, scale=scale, lse=lse.to(dev).contiguous())
    got = out.float().cpu()
    lv = live(acsr_np)
    tol = {torch.float32: 2e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype]   # rounding of values <= 1
    assert float((got - want)[..., lv].abs().max()) <= tol
    assert torch.all(got[..., ~lv] == SENTINEL)


@pytest.mark.parametrize("in_dt,out_dt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                          (torch.float32, torch.bfloat16)])
@pytest.mark.parametrize("make,d", [
    (lambda: O.create_causal_windowed_mask(1024, 511), 64),    # T = 512: rows of whole 16-byte pieces, short rows on top
    (lambda: O.create_causal_windowed_mask(1024, 399), 128),   # T = 400, not a multiple of 64: every row ends inside a line
    (lambda: O.create_windowed_mask(1024, 197), 64),           # T = 395: odd row length, rows clipped at both borders
    (lambda: O.create_dilated_mask(1024, 448, 2), 64),         # row-stride grouping, T = 448
    (lambda: O.create_blocked_mask(1024, 250), 64)],           # T = 500
    ids=["causal512", "causal400", "window395", "dilated448", "blocked500"])
def test_sddmm_line_wise_output(dev, make, d, in_dt, out_dt):
    """Launches with at least 512 row blocks, 16-bit output and T >= 384 collect each row's scores in an LDS ring and
    store whole 64-slot lines: same values as the oracle in every live slot, dead slots untouched."""
    mask = make()
    L = mask.shape[0]
    B, H = 8, 8  # 64 x 8 row blocks = 512
    q, k, _ = O.make_inputs(21, B, H, L, d, in_dt)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    assert acsr[5] >= 384
    scale = d ** -0.5
    out = torch.full((B, H, L, acsr[5]), SENTINEL, dtype=out_dt, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[5], acsr[4],
                            (1, 1), None, None, 16, 16, scale=scale)
    want = O.sddmm(q, k.transpose(2, 3), acsr_np, scale)
    got = out.float().cpu()
    lv = live(acsr_np)
    tol = TOL[out_dt] * max(1.0, float(want.abs().max()))
    assert float((got - want)[..., lv].abs().max()) <= tol
    assert torch.all(got[..., ~lv] == SENTINEL), "dead slots must not be written"


def test_sddmm_line_wise_output_of_short_rows_in_a_large_launch(dev):
    """Rows of four lines (T = 256) take the line-wise path only in launches of at least 4096 row blocks: the 16-bit
    output must be the rounding of what the piece-wise path writes in float32 (same accumulators), dead slots untouched."""
    L, d, B, H = 1024, 64, 16, 32
    pat = A.causal_windowed_pattern(L, 255)
    acsr = A.create_acsr(pat, 16, dev)
    T = acsr[5]
    assert T == 256
    g = torch.Generator().manual_seed(23)
    q = torch.randn(B, H, L, d, generator=g).to(torch.bfloat16).to(dev)
    k = torch.randn(B, H, L, d, generator=g).to(torch.bfloat16).to(dev)
    outs = {}
    for dt in (torch.float32, torch.bfloat16):
        out = torch.full((B, H, L, T), SENTINEL, dtype=dt, device=dev)
        r_sddmm.rsddmm_launcher(q, k.transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4], (1, 1), None, None,
                                16, 16, scale=d ** -0.5)
        outs[dt] = out
    live_slots = torch.arange(T, device=dev)[None, :] < acsr[4][:, None]
    zero = torch.zeros((), dtype=torch.bfloat16, device=dev)
    a, b = outs[torch.float32].to(torch.bfloat16), outs[torch.bfloat16]
    assert torch.equal(torch.where(live_slots, a, zero), torch.where(live_slots, b, zero))
    assert torch.all(b[..., ~live_slots] == SENTINEL)


def test_sddmm_line_wise_output_of_a_long_sequence(dev):
    """L = 2^17 rows of 512 slots through the line-wise path: with q = 1 every score is the sum of its key's
    components, so slot s of row r must hold the column sum of key r - 511 + s (rows above 511: key s)."""
    L, d, w = 1 << 17, 64, 512
    acsr = A.create_acsr(A.causal_windowed_pattern(L, w - 1), 16, dev)
    T = acsr[5]
    g = torch.Generator().manual_seed(24)
    k = torch.randn(1, 1, L, d, generator=g).to(torch.bfloat16).to(dev)
    q = torch.ones(1, 1, L, d, dtype=torch.bfloat16, device=dev)
    out = torch.full((1, 1, L, T), SENTINEL, dtype=torch.bfloat16, device=dev)
    r_sddmm.rsddmm_launcher(q, k.transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4], (1, 1), None, None, 16, 16)
    sums = k.float().sum(-1)[0, 0]                                     # [L]
    rows = torch.arange(L, device=dev)[:, None]
    slots = torch.arange(T, device=dev)[None, :]
    first = torch.clamp(rows - (w - 1), min=0)
    live = slots < torch.clamp(rows + 1, max=w)
    want = sums[torch.clamp(first + slots, max=L - 1)]
    got = out[0, 0].float()
    assert float((got - want)[live].abs().max()) <= 2 ** -7 * float(sums.abs().max()) + 1e-3  # one bf16 rounding
    assert torch.all(got[~live] == SENTINEL)


def test_sddmm_line_wise_output_two_segments(dev):
    """The same path with two segments per row (local window 400 + every 8th earlier column): the second segment's
    slots start at offset 400 of a row of 478."""
    L, d = 1024, 64
    pats = A.strided_patterns(L, 400, 8)
    dms = O.create_strided_segment_masks(L, 400, 8)
    segs = A.create_acsr_segments(pats, 16, dev)
    assert segs.T >= 384 and len(segs) == 2
    B, H = 8, 8
    q, k, _ = O.make_inputs(22, B, H, L, d, torch.bfloat16)
    out = torch.full((B, H, L, segs.T), SENTINEL, dtype=torch.bfloat16, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, None, None, None, None, segs.T, None, None, None, None,
                            16, 16, scale=d ** -0.5, segments=segs)
    dense = (q.float() @ k.float().transpose(2, 3)) * d ** -0.5
    want = torch.cat([O.compress(dense, O.create_acsr(m, 16), first_col=O.row_extents(m)[0], fill=SENTINEL) for m in dms], dim=-1)
    got = out.float().cpu()
    lv = want != SENTINEL
    assert float((got - want)[lv].abs().max()) <= TOL[torch.bfloat16] * max(1.0, float(dense.abs().max()))
    assert torch.all(got[~lv] == SENTINEL)


def _random_rows_mask(L, seed, steps, max_cnt):
    """Rows with a random first column, count and (if `steps` has more than one entry) step; row 3 empty, row 5 a single
    column, one row with exactly `max_cnt` columns."""
    rng = np.random.default_rng(seed)
    m = np.zeros((L, L), np.uint8)
    for r in range(L):
        st = int(rng.choice(steps))
        n = int(rng.integers(0, max_cnt + 1))
        if r == 3:
            n = 0
        if r == 5:
            n = 1
        if r == 7:
            n, st = max_cnt, 1
        a = int(rng.integers(0, L - st * max(n, 1)))
        m[r, a:a + st * n:st] = 1
    return m


MANY_BLOCKS = {
    # d = 128, rows of one or two lines: steps of 64 keys, half lines; L is not a multiple of the row block
    "causal128_d128": (lambda: O.create_causal_windowed_mask(1000, 127), 128),
    # d = 64, rows of one line: half lines
    "causal64_d64": (lambda: O.create_causal_windowed_mask(1000, 63), 64),
    # d = 128, long rows: steps of 32 keys, whole lines; row-stride grouping
    "dilated512_d128": (lambda: O.create_dilated_mask(1024, 512, 2), 128),
    "blocked512_d128": (lambda: O.create_blocked_mask(1024, 256), 128),
    # row-stride grouping with a sequence length that fills neither the last row block nor the last group of two
    "dilated128_L1000_d64": (lambda: O.create_dilated_mask(1000, 256, 2), 64),
    # every row its own span (an empty row, a single-column row): uniform plans whose wavefronts never drop the tests
    "ragged304_d128": (lambda: _random_rows_mask(1024, 31, [1], 304), 128),
    "ragged96_d64": (lambda: _random_rows_mask(1024, 32, [1], 96), 64),
    # rows with differing steps: dense walks, element-wise stores
    "steps200_d64": (lambda: _random_rows_mask(1024, 33, [1, 2, 3], 200), 64),
    "steps200_d128": (lambda: _random_rows_mask(1024, 34, [1, 2, 3], 200), 128),
}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", list(MANY_BLOCKS))
def test_sddmm_16_bit_in_launches_of_many_row_blocks(dev, case, dtype):
    """16-bit SDDMM with d = 64 / 128 and aligned rows (here in launches of 512 row blocks) runs the kernel of thin wavefronts
    (K through an LDS-DMA ring, scores through per-row rings, stores of whole or half lines): every variant it has, on
    uniform and non-uniform plans, against the oracle; dead slots untouched."""
    make, d = MANY_BLOCKS[case]
    mask = make()
    L = mask.shape[0]
    B, H = 8, 8  # 64 x 8 row blocks = 512
    q, k, _ = O.make_inputs(41, B, H, L, d, dtype)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    T = acsr[5]
    assert T % 8 == 0
    scale = d ** -0.5
    out = torch.full((B, H, L, T), SENTINEL, dtype=dtype, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                            (1, 1), None, None, 16, 16, scale=scale)
    want = O.sddmm(q, k.transpose(2, 3), acsr_np, scale, first_col=O.row_extents(mask)[0])
    got = out.float().cpu()
    lv = live(acsr_np)
    tol = TOL[dtype] * max(1.0, float(want.abs().max()))
    assert float((got - want)[..., lv].abs().max()) <= tol
    assert torch.all(got[..., ~lv] == SENTINEL), "dead slots must not be written"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("make,d", [(lambda: O.create_causal_windowed_mask(1000, 255), 128),
                                    (lambda: O.create_dilated_mask(1024, 128, 2), 64)], ids=["causal256_d128", "dilated64_d64"])
def test_sddmm_probabilities_in_launches_of_many_row_blocks(dev, make, d, dtype):
    """The same kernel with a row statistic: exp(scale * score - lse[row]) in the live slots."""
    mask = make()
    L = mask.shape[0]
    B, H = 8, 8
    q, k, _ = O.make_inputs(42, B, H, L, d, dtype)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    T = acsr[5]
    assert T % 8 == 0
    scale = d ** -0.5
    scores = torch.einsum("bhqd,bhkd->bhqk", q.float(), k.float()) * scale
    lse = torch.logsumexp(scores.masked_fill(torch.as_tensor(mask == 0), float("-inf")), dim=-1)
    want = O.softmax_compressed(O.sddmm(q, k.transpose(2, 3), acsr_np, scale), live(acsr_np))
    out = torch.full((B, H, L, T), SENTINEL, dtype=dtype, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                            (1, 1), None, None, 16, 16, scale=scale, lse=lse.to(dev).contiguous())
    got = out.float().cpu()
    lv = live(acsr_np)
    tol = {torch.float16: 1e-3, torch.bfloat16: 8e-3}[dtype]   # rounding of values <= 1
    assert float((got - want)[..., lv].abs().max()) <= tol
    assert torch.all(got[..., ~lv] == SENTINEL)


@pytest.mark.parametrize("case", list(MANY_BLOCKS))
def test_sddmm_with_the_plan_table_equals_sddmm_without(dev, case):
    """By default such launches read the mask's plan table (built on the first call, kept with the metadata); plan=False
    makes every workgroup derive its plan from the ACSR arrays.  Same bits, live and dead slots alike; the table is built
    once per metadata."""
    make, d = MANY_BLOCKS[case]
    mask = make()
    L = mask.shape[0]
    B, H = 8, 8
    q, k, _ = O.make_inputs(44, B, H, L, d, torch.bfloat16)
    acsr = A.create_acsr(mask, 16, dev)
    T = acsr[5]
    outs = []
    for plan in (None, False, None):
        out = torch.full((B, H, L, T), SENTINEL, dtype=torch.bfloat16, device=dev)
        r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                                (1, 1), None, None, 16, 16, scale=d ** -0.5, plan=plan)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    plans = acsr[3].splat_plans
    assert len(plans) == 1


def test_sddmm_refuses_a_plan_that_is_too_small_and_ignores_one_it_has_no_use_for(dev):
    mask = O.create_causal_windowed_mask(1024, 127)
    acsr = A.create_acsr(mask, 16, dev)
    T = acsr[5]
    segs = A.ACSRSegments.single(acsr[0], acsr[1], acsr[2], acsr[3], acsr[4], T)
    plan = segs.plan(1024, dev)
    q, k, _ = O.make_inputs(45, 8, 8, 1024, 64, torch.bfloat16)
    out = torch.empty(8, 8, 1024, T, dtype=torch.bfloat16, device=dev)
    with pytest.raises(Exception, match="plan holds"):
        r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                                (1, 1), None, None, 16, 16, plan=plan[:plan.numel() // 2])
    # float32 takes the general kernel, which has no use for the table: same result with and without
    q32, k32, _ = O.make_inputs(46, 1, 2, 1024, 40, torch.float32)
    a = torch.full((1, 2, 1024, T), SENTINEL, dtype=torch.float32, device=dev)
    b = torch.full_like(a, SENTINEL)
    r_sddmm.rsddmm_launcher(q32.to(dev), k32.to(dev).transpose(2, 3), a, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                            (1, 1), None, None, 16, 16, plan=plan)
    r_sddmm.rsddmm_launcher(q32.to(dev), k32.to(dev).transpose(2, 3), b, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4],
                            (1, 1), None, None, 16, 16, plan=False)
    assert torch.equal(a, b)


def test_the_unfused_launchers_under_stream_capture(dev):
    """A launcher whose first qualifying call happens under stream capture must not build its plan table there (that
    synchronises): it runs without one, and a capture after an eager call uses the table that call left.  Replays equal
    the eager results."""
    mask = O.create_causal_windowed_mask(1024, 255)
    L, d, B, H = 1024, 64, 8, 8
    q, k, v = O.make_inputs(47, B, H, L, d, torch.bfloat16)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    kT = kd.transpose(2, 3)
    outs = []
    for warm in (False, True):
        acsr = A.create_acsr(mask, 16, dev)
        T = acsr[5]
        scores = torch.full((B, H, L, T), SENTINEL, dtype=torch.bfloat16, device=dev)
        o = torch.zeros(B, H, L, d, dtype=torch.bfloat16, device=dev)

        def run():
            r_sddmm.rsddmm_launcher(qd, kT, scores, acsr[0], acsr[1], acsr[2], acsr[3], T, acsr[4], (1, 1), None, None, 16, 16,
                                    scale=d ** -0.5)
            r_softmax.rsoftmax_launcher(scores, scores, acsr[0], acsr[1], acsr[2], acsr[3], T, 256, acsr[4], (1, 1), 16)
            r_spmm.rspmm_launcher(scores, vd, o, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4], (1, 1, 1), 16, 16)
        if warm:
            run()
            assert hasattr(acsr[3], "splat_plans")
        torch.cuda.synchronize()
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                run()
        torch.cuda.current_stream(dev).wait_stream(side)
        assert warm or not hasattr(acsr[3], "splat_plans")
        o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        outs.append(o.clone())
    want = O.dense_masked_attention(q, k.transpose(2, 3), v, np.asarray(mask), d ** -0.5)
    for got in outs:
        assert float((got.float().cpu() - want).abs().max()) <= 2 * TOL[torch.bfloat16]


def test_sddmm_two_aligned_segments_in_a_launch_of_many_row_blocks(dev):
    """Two segments per row whose slots both start on 16-byte boundaries (local window 384 + every 8th earlier column: the
    second segment's slots start at offset 384 of a row of 464): the thin-wavefront kernel walks one segment after the
    other through the same rings."""
    L, d = 1024, 128
    pats = A.strided_patterns(L, 384, 8)
    dms = O.create_strided_segment_masks(L, 384, 8)
    segs = A.create_acsr_segments(pats, 16, dev)
    assert segs.T % 8 == 0 and len(segs) == 2
    B, H = 8, 8
    q, k, _ = O.make_inputs(43, B, H, L, d, torch.bfloat16)
    out = torch.full((B, H, L, segs.T), SENTINEL, dtype=torch.bfloat16, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, None, None, None, None, segs.T, None, None, None, None,
                            16, 16, scale=d ** -0.5, segments=segs)
    dense = (q.float() @ k.float().transpose(2, 3)) * d ** -0.5
    want = torch.cat([O.compress(dense, O.create_acsr(m, 16), first_col=O.row_extents(m)[0], fill=SENTINEL) for m in dms], dim=-1)
    got = out.float().cpu()
    lv = want != SENTINEL
    assert float((got - want)[lv].abs().max()) <= TOL[torch.bfloat16] * max(1.0, float(dense.abs().max()))
    assert torch.all(got[~lv] == SENTINEL)


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("n,p", REF_SMALL)
def test_softmax_reference_cases(dev, n, p):
    """r_softmax.py:188-224 with its masks: fp32 integer-valued input, bf16 output; live slots of every
    row sum to 1 +- 1e-2 (the reference's rule) and match the oracle's values."""
    mask = A.create_blocked_mask(n, p)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    grid, out, full, pow2 = r_softmax.rsoftmax_preamble(mask, (2, 2, n, acsr[5]), 16, dev, torch.bfloat16)
    g = torch.Generator().manual_seed(n + p)
    inp = torch.randint(0, 100, full, generator=g).float()
    out.fill_(SENTINEL)
    res = r_softmax.rsoftmax_launcher(inp.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[5], pow2, acsr[4], grid, 16)
    assert res[0] is out
    lv = live(acsr_np)
    got = out.float().cpu()
    sums = torch.where(lv, got, torch.zeros(())).sum(-1)
    assert torch.all(torch.abs(sums - 1) < 1e-2)
    want = O.softmax_compressed(inp, lv)
    assert float((got - want)[..., lv].abs().max()) <= TOL[torch.bfloat16]
    assert torch.all(got[..., ~lv] == SENTINEL)


@pytest.mark.parametrize("in_dt,out_dt", [(torch.float32, torch.float32), (torch.float16, torch.float16),
                                          (torch.bfloat16, torch.bfloat16), (torch.float32, torch.float16)])
@pytest.mark.parametrize("make", [lambda: O.create_causal_windowed_mask(512, 255), lambda: O.create_windowed_mask(200, 50),
                                  lambda: O.create_dilated_mask(700, 512, 2), lambda: O.create_blocked_mask(3000, 1300)])
def test_softmax_patterns(dev, in_dt, out_dt, make):
    mask = make()
    L = mask.shape[0]
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    T = acsr[5]
    g = torch.Generator().manual_seed(T)
    x = (torch.randn(2, 2, L, T, generator=g) * 3).to(in_dt)
    lv = live(acsr_np)
    want = O.softmax_compressed(x.float(), lv)
    out = torch.full((2, 2, L, T), SENTINEL, dtype=out_dt, device=dev)
    r_softmax.rsoftmax_launcher(x.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], T, O.rsoftmax_pow2(T), acsr[4], (1, 1), 16)
    got = out.float().cpu()
    assert float((got - want)[..., lv].abs().max()) <= TOL[out_dt]
    assert torch.all(got[..., ~lv] == SENTINEL)
    # in place
    xd = x.to(dev)
    if in_dt == out_dt:
        r_softmax.rsoftmax_launcher(xd, xd, acsr[0], acsr[1], acsr[2], acsr[3], T, O.rsoftmax_pow2(T), acsr[4], (1, 1), 16)
        assert float((xd.float().cpu() - want)[..., lv].abs().max()) <= TOL[out_dt]


@pytest.mark.parametrize("in_dt,out_dt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32), (torch.float32, torch.float32)])
@pytest.mark.parametrize("L,w", [(3, 4), (40, 12), (300, 190), (260, 249), (1100, 1000), (2100, 2030), (2100, 2034)])
def test_softmax_row_widths_that_are_not_multiples_of_eight(dev, in_dt, out_dt, L, w):
    """Rows of T = w + 1 slots start anywhere inside an 8-element chunk (T = 191 is config 3's width): every live slot
    matches the oracle, dead slots and the elements after the buffer keep what they held, also in place."""
    mask = O.create_causal_windowed_mask(L, w)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    T = acsr[5]
    assert T == min(L, w + 1) and (T % 8 != 0 or L < 8)
    BH = (3, 1)
    g = torch.Generator().manual_seed(T)
    x = (torch.randn(*BH, L, T, generator=g) * 3).to(in_dt)
    lv = live(acsr_np)
    want = O.softmax_compressed(x.float(), lv)
    n = x.numel()
    buf = torch.full((n + 64,), SENTINEL, dtype=out_dt, device=dev)
    out = buf[:n].view(*BH, L, T)
    r_softmax.rsoftmax_launcher(x.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], T, O.rsoftmax_pow2(T), acsr[4], (1, 1), 16)
    got = out.float().cpu()
    assert float((got - want)[..., lv].abs().max()) <= TOL[out_dt]
    assert torch.all(got[..., ~lv] == SENTINEL)
    assert torch.all(buf[n:] == SENTINEL)
    if in_dt == out_dt:
        inbuf = torch.full((n + 64,), SENTINEL, dtype=in_dt, device=dev)
        xd = inbuf[:n].view(*BH, L, T)
        xd.copy_(x)
        r_softmax.rsoftmax_launcher(xd, xd, acsr[0], acsr[1], acsr[2], acsr[3], T, O.rsoftmax_pow2(T), acsr[4], (1, 1), 16)
        assert float((xd.float().cpu() - want)[..., lv].abs().max()) <= TOL[out_dt]
        assert torch.all(inbuf[n:] == SENTINEL)


# ---------------------------------------------------------------- SpMM
@pytest.mark.parametrize("n,p", REF_SMALL)
def test_spmm_reference_cases(dev, n, p):
    """r_spmm.py:219-261 with its masks: fp32 integer-valued P [.., n, T] and V [.., n, n], every output element
    within 1e-3 of the dot product over live slots (exact here)."""
    mask = A.create_blocked_mask(n, p)
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    g = torch.Generator().manual_seed(n * 7 + p)
    left = torch.randint(0, 100, (2, 2, n, acsr[5]), generator=g).float()
    right = torch.randint(0, 100, (2, 2, n, n), generator=g).float()
    out, grid, T = r_spmm.rspmm_preamble(mask, (2, 2, n, n), 16, 16, dev, torch.float32)
    assert T == acsr[5]
    res = r_spmm.rspmm_launcher(left.to(dev), right.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T,
                                acsr[4], grid, 16, 16)
    assert res[0] is out
    want = O.spmm(left, right, acsr_np)
    assert float((out.cpu() - want).abs().max()) <= 1e-3 * max(1.0, float(want.abs().max()) * 1e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("make,n_out", [
    (lambda: O.create_causal_windowed_mask(512, 63), 64), (lambda: O.create_windowed_mask(300, 20), 40),
    (lambda: O.create_dilated_mask(256, 32, 2), 128), (lambda: O.create_blocked_mask(200, 33), 200),
    (lambda: O.create_causal_windowed_mask(130, 9), 10)])
def test_spmm_patterns(dev, dtype, make, n_out):
    mask = make()
    L = mask.shape[0]
    acsr, acsr_np = acsr_pair(mask, 16, dev)
    T = acsr[5]
    g = torch.Generator().manual_seed(T + n_out)
    lv = live(acsr_np)
    p = torch.rand(2, 3, L, T, generator=g)
    p = (p / torch.where(lv, p, torch.zeros(())).sum(-1, keepdim=True)).to(dtype)
    p = torch.where(lv, p, torch.full((), float("nan"), dtype=dtype))  # dead slots hold garbage
    v = torch.randn(2, 3, L, n_out, generator=g).to(dtype)
    want = O.spmm(torch.nan_to_num(p.float()), v, acsr_np)
    out = torch.empty(2, 3, L, n_out, dtype=dtype, device=dev)
    r_spmm.rspmm_launcher(p.to(dev), v.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4],
                          (1, 1, 1), 16, 16)
    assert float((out.float().cpu() - want).abs().max()) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n_out", [64, 128])
@pytest.mark.parametrize("make", [
    lambda: [A.causal_windowed_pattern(700, 199)], lambda: [A.windowed_pattern(513, 130)], lambda: [A.dilated_pattern(640, 96, 2)],
    lambda: [A.blocked_pattern(512, 128)], lambda: A.strided_patterns(768, 64, 32), lambda: [A.causal_windowed_pattern(100, 5)]],
    ids=["causal window", "window", "dilated", "blocked", "strided, two segments", "rows shorter than a piece"])
def test_spmm_16_bit_whole_rows_of_v(dev, make, n_out, dtype):
    """16-bit operands with 64 or 128 output columns (one workgroup takes whole rows of V): several row blocks and tiles,
    a last block that is not full, spans that end inside tiles, gathered keys, two segments, rows with fewer live slots than
    one 16-byte piece; dead slots hold NaN and must not reach the output."""
    pats = make()
    L = pats[0].s
    segs = A.create_acsr_segments(pats, 16, dev)
    dms = [np.asarray(pt.device_mask(dev).cpu()) for pt in pats]
    T = segs.T
    g = torch.Generator().manual_seed(T + n_out)
    lv = torch.cat([torch.from_numpy(O.slot_columns(O.create_acsr(m, 16))[1]) for m in dms], dim=-1)
    pr = torch.rand(2, 2, L, T, generator=g)
    pr = (pr / torch.where(lv, pr, torch.zeros(())).sum(-1, keepdim=True).clamp(min=1e-9)).to(dtype)
    pr = torch.where(lv, pr, torch.full((), float("nan"), dtype=dtype))
    v = torch.randn(2, 2, L, n_out, generator=g).to(dtype)
    dense = torch.zeros(2, 2, L, L)
    off = 0
    for m in dms:
        acsr_np = O.create_acsr(m, 16)
        cols, valid = O.slot_columns(acsr_np, first_col=O.row_extents(m)[0])
        Tk = cols.shape[-1]
        blk = torch.nan_to_num(pr[..., off:off + Tk].float())
        rows_i, slots_i = np.nonzero(valid)
        dense[:, :, torch.from_numpy(rows_i), torch.from_numpy(cols[rows_i, slots_i].astype(np.int64))] += blk[:, :, torch.from_numpy(rows_i), torch.from_numpy(slots_i)]
        off += Tk
    want = dense @ v.float()
    out = torch.full((2, 2, L, n_out), 7.0, dtype=dtype, device=dev)
    r_spmm.rspmm_launcher(pr.to(dev), v.to(dev), out, None, None, None, None, None, None, T, None, None, 16, 16, segments=segs)
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert float((got - want).abs().max()) <= TOL[dtype]


def _spmm_case(mask, n_out, dtype, B=8, H=8, seed=51):
    """Probabilities (NaN in the dead slots), V and the dense fp32 answer for one mask."""
    L = mask.shape[0]
    acsr_np = O.create_acsr(mask, 16)
    cols, valid = O.slot_columns(acsr_np, first_col=O.row_extents(mask)[0])
    T = cols.shape[-1]
    lv = torch.from_numpy(valid)
    g = torch.Generator().manual_seed(seed + n_out)
    pr = torch.rand(B, H, L, T, generator=g)
    pr = (pr / torch.where(lv, pr, torch.zeros(())).sum(-1, keepdim=True).clamp(min=1e-9)).to(dtype)
    pr = torch.where(lv, pr, torch.full((), float("nan"), dtype=dtype))
    v = torch.randn(B, H, L, n_out, generator=g).to(dtype)
    dense = torch.zeros(B, H, L, L)
    rows_i, slots_i = np.nonzero(valid)
    ri, si = torch.from_numpy(rows_i), torch.from_numpy(slots_i)
    dense[:, :, ri, torch.from_numpy(cols[rows_i, slots_i].astype(np.int64))] = torch.nan_to_num(pr.float())[:, :, ri, si]
    return pr, v, dense @ v.float(), T


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", list(MANY_BLOCKS))
def test_spmm_16_bit_in_launches_of_many_row_blocks(dev, case, dtype):
    """16-bit SpMM with 64 / 128 output columns, here in launches of 512 row blocks: with the mask's plan table (the default unless
    the rows are long and every one starts on a multiple of 8 positions) the kernels that start from it run -- rows of
    fewer than 256 slots through a workgroup-wide tile, longer ones through per-row rings or, where they start on 16-byte
    boundaries, straight from memory; spans that end inside half steps, rows that are empty or hold one column, rows with
    differing steps -- and must agree with the dense product; dead slots hold NaN and must not reach the output; the
    general kernel (plan=False) must agree too."""
    make, d = MANY_BLOCKS[case]
    mask = make()
    L = mask.shape[0]
    pr, v, want, T = _spmm_case(mask, d, dtype)
    acsr = A.create_acsr(mask, 16, dev)
    assert acsr[5] == T
    outs = []
    for plan in (None, False):
        out = torch.full((8, 8, L, d), 7.0, dtype=dtype, device=dev)
        r_spmm.rspmm_launcher(pr.to(dev), v.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4],
                              (1, 1, 1), 16, 16, plan=plan)
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        assert float((got - want).abs().max()) <= TOL[dtype]
        outs.append(got)
    assert float((outs[0] - outs[1]).abs().max()) <= TOL[dtype] / 4
    segs = A.ACSRSegments.single(acsr[0], acsr[1], acsr[2], acsr[3], acsr[4], T)
    assert segs.plan_is_aligned(L, dev) == case.startswith("blocked")


def test_spmm_with_a_plan_forced_on_an_aligned_mask_and_two_segments(dev):
    """A blocked mask takes the general kernel by default; given its plan explicitly it runs the thin wavefronts, whose
    rows then read their aligned chunks straight from memory.  Two aligned segments per row go one after the other."""
    mask = O.create_blocked_mask(1024, 256)
    pr, v, want, T = _spmm_case(mask, 128, torch.bfloat16, seed=52)
    acsr = A.create_acsr(mask, 16, dev)
    segs = A.ACSRSegments.single(acsr[0], acsr[1], acsr[2], acsr[3], acsr[4], T)
    out = torch.full((8, 8, 1024, 128), 7.0, dtype=torch.bfloat16, device=dev)
    r_spmm.rspmm_launcher(pr.to(dev), v.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4],
                          (1, 1, 1), 16, 16, plan=segs.plan(1024, dev))
    assert float((out.float().cpu() - want).abs().max()) <= TOL[torch.bfloat16]
    with pytest.raises(Exception, match="plan holds"):
        r_spmm.rspmm_launcher(pr.to(dev), v.to(dev), out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4],
                              (1, 1, 1), 16, 16, plan=segs.plan(1024, dev)[:4096])
    # two segments
    L, d = 1024, 64
    pats = A.strided_patterns(L, 384, 8)
    dms = O.create_strided_segment_masks(L, 384, 8)
    segs2 = A.create_acsr_segments(pats, 16, dev)
    parts = [_spmm_case(m, d, torch.float16, seed=53 + i) for i, m in enumerate(dms)]
    pr2 = torch.cat([pt[0] for pt in parts], dim=-1)
    v2 = parts[0][1]
    dense = torch.zeros(8, 8, L, L)
    off = 0
    for m, pt in zip(dms, parts):
        cols, valid = O.slot_columns(O.create_acsr(m, 16), first_col=O.row_extents(m)[0])
        rows_i, slots_i = np.nonzero(valid)
        ri, si = torch.from_numpy(rows_i), torch.from_numpy(slots_i)
        dense[:, :, ri, torch.from_numpy(cols[rows_i, slots_i].astype(np.int64))] += torch.nan_to_num(pt[0].float())[:, :, ri, si]
    want2 = dense @ v2.float()
    assert pr2.shape[-1] == segs2.T
    out2 = torch.full((8, 8, L, d), 7.0, dtype=torch.float16, device=dev)
    r_spmm.rspmm_launcher(pr2.to(dev), v2.to(dev), out2, None, None, None, None, None, None, segs2.T, None, None, 16, 16,
                          segments=segs2)
    got2 = out2.float().cpu()
    assert torch.isfinite(got2).all()
    assert float((got2 - want2).abs().max()) <= 2 * TOL[torch.float16]


@pytest.mark.parametrize("case", ["dilated512x2_d128_bf16", "causal511_d64_f16", "blocked512_d128_bf16"])
def test_spmm_rings_on_a_compressed_matrix_larger_than_the_last_level_cache(dev, case):
    """Rows of at least 256 slots on 16-byte boundaries and more than 192 MB of probabilities (here 268 MB) take the kernel of
    per-row rings, whose lines are loaded non-temporally; on a blocked mask (the table passed by hand: the launcher would
    pick the general kernel) its wavefronts read aligned chunks straight from memory.  Against the general kernel over the
    whole output and against the dense product for two (batch, head) pairs; dead slots hold NaN."""
    make, d, dtype = {"dilated512x2_d128_bf16": (lambda: O.create_dilated_mask(4096, 512, 2), 128, torch.bfloat16),
                      "causal511_d64_f16": (lambda: O.create_causal_windowed_mask(4096, 511), 64, torch.float16),
                      "blocked512_d128_bf16": (lambda: O.create_blocked_mask(4096, 256), 128, torch.bfloat16)}[case]
    mask = make()
    L, B, H = mask.shape[0], 8, 8
    acsr_np = O.create_acsr(mask, 16)
    cols, valid = O.slot_columns(acsr_np, first_col=O.row_extents(mask)[0])
    T = cols.shape[-1]
    assert T == 512 and B * H * L * T * 2 > (192 << 20)
    lv = torch.from_numpy(valid).to(dev)
    g = torch.Generator(device=dev).manual_seed(71)
    pr = torch.rand(B, H, L, T, generator=g, device=dev)
    pr = pr / torch.where(lv, pr, torch.zeros((), device=dev)).sum(-1, keepdim=True).clamp(min=1e-9)
    pr = torch.where(lv, pr, torch.full((), float("nan"), device=dev)).to(dtype)
    v = torch.randn(B, H, L, d, generator=g, device=dev).to(dtype)
    acsr = A.create_acsr(mask, 16, dev)
    segs = A.ACSRSegments.single(acsr[0], acsr[1], acsr[2], acsr[3], acsr[4], T)
    outs = []
    for plan in (segs.plan(L, dev), False):
        out = torch.full((B, H, L, d), 7.0, dtype=dtype, device=dev)
        r_spmm.rspmm_launcher(pr, v, out, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7], T, acsr[4],
                              (1, 1, 1), 16, 16, plan=plan)
        assert torch.isfinite(out).all()
        outs.append(out.float())
    assert float((outs[0] - outs[1]).abs().max()) <= TOL[dtype]
    rows_i, slots_i = np.nonzero(valid)
    ri, si = torch.from_numpy(rows_i).to(dev), torch.from_numpy(slots_i).to(dev)
    ci = torch.from_numpy(cols[rows_i, slots_i].astype(np.int64)).to(dev)
    for b, h in ((0, 0), (B - 1, H - 1)):
        dense = torch.zeros(L, L, device=dev)
        dense[ri, ci] = pr[b, h].float()[ri, si]
        assert float((outs[0][b, h] - dense @ v[b, h].float()).abs().max()) <= TOL[dtype]


def test_comparison_sweeps_run_and_agree_with_dense(dev):
    """The sweep harness (successor of the reference's comparison.py:76-106) at toy size: one record per doubling of
    the sparsity parameter, nnz as the pattern's closed form, fused forward equal to dense attention with the same mask."""
    import comparison
    rows = comparison.benchmark("Windowed", 64, 16, 16, dev, verbose=False)
    assert [r["sparsity_parameter"] for r in rows] == [2, 4, 8, 16, 32, 64]
    for r in rows:
        p = r["sparsity_parameter"]
        assert r["nnz"] == sum(min(63, i + p) - max(0, i - p) + 1 for i in range(64))
        assert r["splat_ms"] > 0 and r["dense_ms"] > 0
    att = comparison.benchmark_attention("Blocked", 128, dev, batch=1, num_heads=2, head_dim=64, dtype=torch.float16,
                                         verbose=False)
    assert len(att) == 7 and max(r["max_abs_diff"] for r in att) <= 1e-2
    with pytest.raises(Exception, match="Not implemented!"):
        comparison.benchmark("Strided", 64, 16, 16, dev, verbose=False)


def test_a_segment_that_is_empty_everywhere_is_dropped(dev):
    """Strided pattern on a sequence shorter than its local window: the far segment has no column at all."""
    segs = A.create_acsr_segments(A.strided_patterns(100, 128, 16), 16, dev)
    assert len(segs) == 1 and segs.T == 100
    q, k, _ = O.make_inputs(3, 1, 2, 100, 64, torch.float32)
    out = torch.zeros(1, 2, 100, segs.T, device=dev)
    r_sddmm.rsddmm_launcher(q.to(dev), k.to(dev).transpose(2, 3), out, None, None, None, None, segs.T, None, None, None, None,
                            16, 16, segments=segs)
    want = torch.tril(q @ k.transpose(2, 3))
    got = out.cpu()
    for r in (0, 37, 99):
        assert float((got[0, 1, r, :r + 1] - want[0, 1, r, :r + 1]).abs().max()) <= 1e-4


@pytest.mark.parametrize("n_bytes", [16, 4096 * 16, (4096 * 3 + 1000) * 16 + 48, 64 << 20])
def test_stream_copy_copies(dev, n_bytes):
    """splat_bench_stream_copy, the streaming ceiling bench.py quotes the softmax against, is a faithful copy: whole
    chunks and the tail that does not fill one, and nothing past the end."""
    import _splat_hip as hip
    import bench_probes as BP
    g = torch.Generator().manual_seed(n_bytes % 1000)
    src = torch.randint(0, 256, (n_bytes + 64,), dtype=torch.uint8, generator=g).to(dev)
    dst = torch.full((n_bytes + 64,), 7, dtype=torch.uint8, device=dev)
    BP.check(BP.lib().splat_bench_stream_copy(src.data_ptr(), dst.data_ptr(), n_bytes, hip.stream_ptr(dev)), "splat_bench_stream_copy")
    assert torch.equal(dst[:n_bytes], src[:n_bytes])
    assert torch.all(dst[n_bytes:] == 7)
    assert BP.lib().splat_bench_stream_copy(src.data_ptr(), dst.data_ptr(), 24, None) == -2
    assert BP.lib().splat_bench_stream_copy(src.data_ptr() + 8, dst.data_ptr(), 32, None) == -4


@pytest.mark.parametrize("shape", [0, 1, 2])
def test_mfma_lds_probe_runs_and_checks_its_arguments(dev, shape):
    """splat_bench_mfma_lds_probe, the matrix loops bench.py quotes the fused forward against: every workgroup computes
    the same figures from the same 64 KiB, zeros give zeros, two calls agree, and short buffers are refused."""
    import _splat_hip as hip
    import bench_probes as BP
    data = torch.randn(32768, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(dev)
    wgs, tiles, nt = 6, 3, BP.PROBE_THREADS[shape]
    out = torch.full((wgs * nt + 8,), 7.0, dtype=torch.float32, device=dev)
    fn = BP.lib().splat_bench_mfma_lds_probe
    call = lambda d, o, w=wgs, t=tiles: fn(d.data_ptr(), d.numel() * 2, o.data_ptr(), wgs * nt * 4, shape, w, t, hip.stream_ptr(dev))
    BP.check(call(data, out), "splat_bench_mfma_lds_probe")
    res = out[:wgs * nt].view(wgs, nt)
    assert torch.isfinite(res).all() and float(res.abs().max()) > 0
    assert torch.equal(res, res[0].expand_as(res))
    assert torch.all(out[wgs * nt:] == 7.0)
    again = torch.empty_like(out)
    BP.check(call(data, again), "splat_bench_mfma_lds_probe")
    assert torch.equal(again[:wgs * nt], out[:wgs * nt])
    BP.check(call(torch.zeros_like(data), again), "splat_bench_mfma_lds_probe")
    assert torch.all(again[:wgs * nt] == 0)
    assert fn(data.data_ptr(), 65535, out.data_ptr(), wgs * nt * 4, shape, wgs, tiles, None) == -2
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4 - 1, shape, wgs, tiles, None) == -2
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4, shape, 0, tiles, None) == -2
    assert fn(data.data_ptr() + 2, 65536, out.data_ptr(), wgs * nt * 4, shape, wgs, tiles, None) == -4
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4, 3, wgs, tiles, None) == -5
    rows = 256 if shape == 1 else 128
    assert BP.lib().splat_bench_mfma_lds_probe_flops(shape, wgs, tiles) == wgs * tiles * rows * 64 * 128 * 4
    assert BP.lib().splat_bench_mfma_lds_probe_flops(3, wgs, tiles) == 0


@pytest.mark.parametrize("exponentials", [1, 0])
@pytest.mark.parametrize("shape", [0, 1])
def test_softmax_loop_probe_runs_and_checks_its_arguments(dev, shape, exponentials):
    """splat_bench_softmax_loop_probe, the d = 64 tile loop with its exponentials that bench.py quotes configs 2 and 3
    against: every workgroup computes the same finite figures from the same data, two calls agree, nothing is written past
    the workgroups' floats, and short buffers are refused."""
    import _splat_hip as hip
    import bench_probes as BP
    data = (0.5 * torch.randn(32768, generator=torch.Generator().manual_seed(6))).to(torch.bfloat16).to(dev)
    wgs, tiles, nt = 5, 3, BP.SOFTMAX_LOOP_THREADS[shape]
    out = torch.full((wgs * nt + 8,), 7.0, dtype=torch.float32, device=dev)
    fn = BP.lib().splat_bench_softmax_loop_probe
    call = lambda d, o: fn(d.data_ptr(), d.numel() * 2, o.data_ptr(), wgs * nt * 4, shape, exponentials, wgs, tiles, hip.stream_ptr(dev))
    BP.check(call(data, out), "splat_bench_softmax_loop_probe")
    res = out[:wgs * nt].view(wgs, nt)
    assert torch.isfinite(res).all() and float(res.abs().max()) > 0
    assert torch.equal(res, res[0].expand_as(res))
    assert torch.all(out[wgs * nt:] == 7.0)
    again = torch.empty_like(out)
    BP.check(call(data, again), "splat_bench_softmax_loop_probe")
    assert torch.equal(again[:wgs * nt], out[:wgs * nt])
    assert fn(data.data_ptr(), 65535, out.data_ptr(), wgs * nt * 4, shape, exponentials, wgs, tiles, None) == -2
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4 - 1, shape, exponentials, wgs, tiles, None) == -2
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4, shape, exponentials, 0, tiles, None) == -2
    assert fn(data.data_ptr() + 2, 65536, out.data_ptr(), wgs * nt * 4, shape, exponentials, wgs, tiles, None) == -4
    assert fn(data.data_ptr(), 65536, out.data_ptr(), wgs * nt * 4, 2, exponentials, wgs, tiles, None) == -5
    assert BP.lib().splat_bench_softmax_loop_probe_flops(wgs, tiles) == wgs * tiles * 128 * 64 * 64 * 4


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("L,d", [(64, 64), (1000, 128), (333, 64), (77, 40), (130, 7), (1, 128)])
def test_key_transpose(dev, L, d, dtype):
    """K^T with the keys contiguous -> K with rows contiguous, bit for bit: whole tensors, a slice of a wider one (longer
    stride of the d index), and a source that starts off a 16-byte boundary (element loads)."""
    B, H = 2, 3
    g = torch.Generator().manual_seed(L * 131 + d)
    wide = torch.randn(B, H, d, L + 24, generator=g).to(dtype).to(dev)
    for kT in (wide[..., :L].contiguous(), wide[..., 8:8 + L], wide[..., 3:3 + L]):
        got = A.transpose_keys(kT)
        assert got.is_contiguous() and tuple(got.shape) == (B, H, L, d)
        assert torch.equal(got, kT.transpose(2, 3).contiguous())
