"""splat_attention_fwd_noalloc (the forward whose plan lives in a buffer built into the library, for callers that
cannot allocate) against splat_attention_fwd_planned, through the C ABI: bit-identical outputs on two calls in a row,
the second on a smaller input, so that what the first call left in the shared buffer is seen not to matter."""
import pytest
import torch

import acsr_helpers as A
import _splat_hip as hip
from r_attention import attention_plan

pytestmark = pytest.mark.gpu


def forward_args(q, kT, v, out, arr, n_seg, scale):
    B, H, L, d = q.shape
    qs, ks, vs, os_ = q.stride(), kT.stride(), v.stride(), out.stride()
    return (q.data_ptr(), qs[0], qs[1], qs[2], kT.data_ptr(), ks[0], ks[1], ks[2], ks[3], v.data_ptr(), vs[0], vs[1], vs[2],
            out.data_ptr(), os_[0], os_[1], os_[2], arr, n_seg, B, H, L, d, float(scale), hip.dtype_code(q.dtype))


def run_pair(dev, patterns, B, H, L, d, dtype, seed):
    g = torch.Generator(device="cpu").manual_seed(seed)
    q, k, v = (torch.randn(B, H, L, d, generator=g).to(dtype).to(dev) for _ in range(3))
    kT = k.transpose(2, 3)
    segs = A.create_acsr_segments(patterns, 16, dev)
    arr = hip.seg_array(segs.seg_args(), L)
    plan = attention_plan(segs, L, dev)
    want = torch.full((B, H, L, d), float("nan"), dtype=dtype, device=dev)
    got = torch.full((B, H, L, d), float("nan"), dtype=dtype, device=dev)
    lib, st = hip.lib(), hip.stream_ptr(dev)
    torch.cuda.synchronize()
    allocated = torch.cuda.memory_allocated(dev)
    rc = lib.splat_attention_fwd_planned(*forward_args(q, kT, v, want, arr, len(segs), d ** -0.5), plan.data_ptr(),
                                         plan.numel(), st)
    hip.check(rc, "splat_attention_fwd_planned")
    rc = lib.splat_attention_fwd_noalloc(*forward_args(q, kT, v, got, arr, len(segs), d ** -0.5), st)
    hip.check(rc, "splat_attention_fwd_noalloc")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) == allocated
    assert not torch.isnan(want.float()).any()
    assert torch.equal(got.view(torch.int16 if dtype != torch.float32 else torch.int32),
                       want.view(torch.int16 if dtype != torch.float32 else torch.int32))


def test_noalloc_forward_matches_the_planned_forward_twice_in_a_row(dev):
    # the larger input first: its plan fills more of the shared buffer than the second call rewrites
    run_pair(dev, A.strided_patterns(2048, 128, 128), 2, 3, 2048, 64, torch.bfloat16, 1)
    run_pair(dev, [A.causal_windowed_pattern(640, 100)], 1, 2, 640, 128, torch.float16, 2)
    run_pair(dev, [A.dilated_pattern(300, 32, 2)], 1, 1, 300, 64, torch.float32, 3)


def test_noalloc_forward_rejects_a_plan_beyond_its_buffer(dev):
    L = 1 << 18
    segs = A.create_acsr_segments([A.causal_windowed_pattern(L, 3)], 16, dev)
    arr = hip.seg_array(segs.seg_args(), L)
    q = torch.zeros(1, 1, L, 64, dtype=torch.float16, device=dev)
    rc = hip.lib().splat_attention_fwd_noalloc(*forward_args(q, q.transpose(2, 3), q, q, arr, 1, 1.0), hip.stream_ptr(dev))
    assert rc == -2
    with pytest.raises(hip.SplatError, match="built-in buffer"):
        hip.check(rc, "splat_attention_fwd_noalloc")


def test_noalloc_forward_replays_from_a_captured_graph_after_another_mask_used_the_buffer(dev):
    """Captured after one eager warm-up call (the first call on a device resolves the built-in buffer's address, which is
    not a stream operation).  Between capture and replays an eager call with another mask overwrites the shared plan
    buffer; a replay rebuilds its own plan first, so every replay must equal the planned forward on the same inputs."""
    B, H, L, d, dtype = 2, 2, 520, 128, torch.bfloat16
    segs = A.create_acsr_segments([A.causal_windowed_pattern(L, 150)], 16, dev)
    arr = hip.seg_array(segs.seg_args(), L)
    plan = attention_plan(segs, L, dev)
    other = A.create_acsr_segments(A.strided_patterns(1024, 64, 64), 16, dev)
    arr_o = hip.seg_array(other.seg_args(), 1024)
    g = torch.Generator().manual_seed(21)
    q, k, v = (torch.randn(B, H, L, d, generator=g).to(dtype).to(dev) for _ in range(3))
    q2, k2, v2 = (torch.randn(1, 1, 1024, d, generator=g).to(dtype).to(dev) for _ in range(3))
    out_g, want, junk = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q2)
    lib = hip.lib()
    noalloc = lambda st: hip.check(lib.splat_attention_fwd_noalloc(*forward_args(q, k.transpose(2, 3), v, out_g, arr, 1, d ** -0.5), st),
                                   "splat_attention_fwd_noalloc")
    noalloc(hip.stream_ptr(dev))                                # warm-up, eager
    torch.cuda.synchronize()
    side = torch.cuda.Stream(device=dev)
    side.wait_stream(torch.cuda.current_stream(dev))
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            noalloc(hip.stream_ptr(dev))
    torch.cuda.current_stream(dev).wait_stream(side)
    for seed in (1, 2, 3):
        gen = torch.Generator().manual_seed(seed)
        for t in (q, k, v):
            t.copy_(torch.randn(B, H, L, d, generator=gen).to(dtype))
        # another mask's call leaves its plan in the shared buffer
        hip.check(lib.splat_attention_fwd_noalloc(*forward_args(q2, k2.transpose(2, 3), v2, junk, arr_o, len(other), 0.1),
                                                  hip.stream_ptr(dev)), "splat_attention_fwd_noalloc")
        torch.cuda.synchronize()
        out_g.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        hip.check(lib.splat_attention_fwd_planned(*forward_args(q, k.transpose(2, 3), v, want, arr, 1, d ** -0.5), plan.data_ptr(),
                                                  plan.numel(), hip.stream_ptr(dev)), "splat_attention_fwd_planned")
        torch.cuda.synchronize()
        assert torch.equal(out_g.view(torch.int16), want.view(torch.int16)), seed
