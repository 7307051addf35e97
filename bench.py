#!/usr/bin/env python3
"""Benchmark of the ACSR sparse-attention forward on one MI355X.

A step is one fused forward (RegularAttention.forward -> splat_attention_fwd_planned, the mask's plan built once in
the untimed set-up like the ACSR arrays) over benchmark configuration 5: B=4, H=16, L=16384, d=128,
bf16, causal window 512, scale 1/sqrt(d), seeded synthetic N(0,1) inputs already resident in HBM, K handed
over as ``k.transpose(2, 3)`` (a view of row-major K; the K^T-contiguous layout is timed as an extra).
Prints ONE JSON line.  `value` counts only nonzero (live) FLOPs: 4 * d * nnz * B * H.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-extras]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "triton-fun_amd", "SPLAT"), os.path.join(ROOT, "triton-fun_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16/fp16
FP32_MFMA_PEAK_TFLOPS = 157.3
HBM_PEAK_GBPS = 8000.0
# HBM bytes one fused launch moves at config 5 are not something this script can measure (hardware counters need
# rocprofv3): the figure comes from the committed counter summary, which names the commit whose kernel it profiled.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "attn_fwd_kernel_cfg5_hbm_traffic.md")
# The GPU's clock takes some tens of launches to settle under this kernel (the first launches of a process run at the
# idle boost clock, the next ones slower, then the steady state): an untimed, declared phase ahead of --warmup.
SETTLE_MIN_LAUNCHES = 100
SETTLE_MIN_MS = 50.0


def profiled_traffic():
    """(bytes per launch, commit) from the lines `traffic_bytes_per_launch: X` / `kernel_commit: Y` of the committed
    counter summary; (None, None) when it is missing or holds no such line."""
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    import re
    b = re.search(r"traffic_bytes_per_launch:\s*([0-9.eE+]+)", text)
    c = re.search(r"kernel_commit:\s*([0-9a-f]+)", text)
    return (float(b.group(1)) if b else None), (c.group(1) if c else None)


FUSED_KERNEL_NAME = "attn_fwd_kernel<bf16, D=128, KT=false, BN=64, NSTAGE=2, PLANNED=true>"


def causal_window_nnz(L: int, w: int) -> int:
    return w * L - w * (w - 1) // 2


def settle(fn):
    """Untimed launches until the clock has settled: at least SETTLE_MIN_LAUNCHES and at least SETTLE_MIN_MS of
    device time.  Returns the number of launches."""
    import torch
    n = 0
    t0 = time.perf_counter()
    while n < SETTLE_MIN_LAUNCHES or (time.perf_counter() - t0) * 1e3 < SETTLE_MIN_MS:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        n += 20
    return n


def time_launches(fn, steps: int, warmup: int):
    """Whole-region wall time (synchronise on both sides) and per-launch HIP-event durations on the
    current stream, in ms."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per = sorted(a.elapsed_time(b) for a, b in evs)
    return wall_ms, per


def time_batch(fn, steps: int, warmup: int) -> float:
    """Mean device time per launch in ms of `steps` back-to-back launches (one event pair around all of them): for kernels
    so short that a per-launch event pair would mostly time the gaps between launches."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def time_cold_launches(fn, scratch, steps: int):
    """Mean per-launch HIP-event duration in ms with a write of `scratch` (larger than L2 + MALL) before every launch,
    so that no launch finds its operands in a cache."""
    import torch
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    for a, b in evs:
        scratch.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in evs) / steps


def sample_power_and_clock(fn, launches_per_batch: int = 50):
    """Socket power (W) and graphics clock (MHz) as `amd-smi metric -p -c` reports them while `fn` is launched back to
    back: two readings at least a second into the loop, averaged.  None when the tool is missing or prints no figures."""
    import re
    import shutil
    import subprocess
    import threading

    import torch

    tool = shutil.which("amd-smi")
    if tool is None:
        return None
    readings, done = [], threading.Event()

    def reader():
        try:
            time.sleep(1.0)
            for _ in range(2):
                txt = subprocess.run([tool, "metric", "-p", "-c"], capture_output=True, text=True, timeout=10).stdout
                pw = re.search(r"SOCKET_POWER:\s*([0-9.]+)\s*W", txt)
                ck = re.search(r"GFX_0:\s*\n\s*CLK:\s*([0-9.]+)\s*MHz", txt)
                if pw and ck:
                    readings.append((float(pw.group(1)), float(ck.group(1))))
        except Exception:
            pass
        finally:
            done.set()

    th = threading.Thread(target=reader, daemon=True)
    th.start()
    t_end = time.perf_counter() + 30.0
    while not done.is_set() and time.perf_counter() < t_end:
        for _ in range(launches_per_batch):
            fn()
        torch.cuda.synchronize()
    th.join(timeout=15.0)
    if not readings:
        return None
    return {"socket_power_w": round(sum(r[0] for r in readings) / len(readings), 1),
            "gfx_clk_mhz": round(sum(r[1] for r in readings) / len(readings), 1),
            "source": "amd-smi metric -p -c, two readings during a sustained loop of the kernel"}


def make_inputs(seed: int, B: int, H: int, L: int, d: int, dtype):
    """Seeded q, k, v ~ N(0,1), drawn in fp32 on the host in that order, then cast."""
    import torch
    g = torch.Generator("cpu").manual_seed(seed)
    return tuple(torch.randn(B, H, L, d, generator=g, dtype=torch.float32).to(dtype) for _ in range(3))


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50,
                    help="untimed launches before the timed ones (the GPU clock needs some tens of launches to settle)")
    ap.add_argument("--no-settle", action="store_true",
                    help="profiling runs: skip the clock-settle phase and the unsettled pass, so that a counter run sees "
                         "only --warmup + --steps launches of the headline kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host baseline")
    ap.add_argument("--no-extras", action="store_true", help="skip the unfused kernels and the ACSR build")
    ap.add_argument("--cpu-heads", type=int, default=16, help="(batch, head) pairs the host baseline computes")
    ap.add_argument("--zero-operands", action="store_true",
                    help="power / clock studies only: q, k and v are all zeros (no switching in the multipliers), which says how "
                         "much of the time is the power limit's; the line is marked and is not a result")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy, the known-size kernel that HBM counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the path shards over batch*heads with no exchange, and this build "
              "has no multi-GPU launcher (--gpus must be 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    import _splat_hip as hip
    import acsr_helpers as A
    import r_softmax
    import r_sddmm
    import r_spmm
    from r_attention import RegularAttention, attention_launcher

    if not torch.cuda.is_available():
        print("bench.py needs a HIP device", file=sys.stderr)
        return 2
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)

    B, H, L, d, w = 4, 16, 16384, 128, 512
    dtype = torch.bfloat16
    scale = d ** -0.5
    q, k, v = make_inputs(1005, B, H, L, d, dtype)
    qd, kd, vd = q.to(dev), k.to(dev), v.to(dev)
    if args.zero_operands:
        qd.zero_(), kd.zero_(), vd.zero_()
    kT_view = kd.transpose(2, 3)

    t0 = time.perf_counter()
    attn = RegularAttention(B, L, H, d, A.causal_windowed_pattern(L, w - 1), 16, 16, dev, dtype, scale=scale)
    torch.cuda.synchronize()
    setup_ms = (time.perf_counter() - t0) * 1e3

    nnz = causal_window_nnz(L, w)
    flops = 4.0 * d * nnz * B * H
    io_bytes = 4.0 * B * H * L * d * 2

    step = lambda: attn([qd, kT_view, vd])
    # what the same --warmup / --steps give in a process that has just started (the clock has not settled)
    cold_wall_ms, cold_per = (0.0, [0.0]) if args.no_settle else time_launches(step, args.steps, args.warmup)
    settle_launches = 0 if args.no_settle else settle(step)
    wall_ms, per = time_launches(step, args.steps, args.warmup)
    ms_per_step = wall_ms / args.steps
    kern_ms = sum(per) / len(per)
    tflops = flops / (ms_per_step * 1e-3) / 1e12
    kern_tflops = flops / (kern_ms * 1e-3) / 1e12

    traffic, traffic_commit = profiled_traffic()
    out = {
        "metric": "sparse-attn fwd ms + nnz-TFLOP/s (% MFMA peak) on 1 MI355X; softmax HBM GB/s",
        "value": round(tflops, 2),
        "unit": "TFLOP/s (nonzero FLOPs only, fused forward)",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "settle_launches": settle_launches,
        "ms_per_step": round(ms_per_step, 4),
        "unsettled": {"ms_per_step": round(cold_wall_ms / args.steps, 4),
                      "kernel_ms_avg": round(sum(cold_per) / len(cold_per), 4),
                      "note": "the same warmup + steps run first, in the just-started process, before the settle phase"},
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": ("ALL-ZERO q/k/v (--zero-operands: a power study, not a result)" if args.zero_operands else
                 "synthetic: seeded N(0,1) q/k/v (torch.Generator cpu seed 1005), resident in HBM"),
        "config": {"workload": "config 5: fused ACSR attention fwd, B=4 H=16 L=16384 d=128 bf16, causal window 512, "
                               "scale 1/sqrt(d), K passed as k.transpose(2,3)",
                   "B": B, "H": H, "L": L, "d": d, "window": w, "nnz_per_head": nnz},
        "roofline": {"bound": "mfma", "achieved": round(kern_tflops, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(kern_tflops / MFMA_PEAK_TFLOPS, 4), "traffic": traffic,
                     "traffic_source": {"profile": os.path.relpath(TRAFFIC_PROFILE, ROOT), "kernel_commit": traffic_commit},
                     "kernel": FUSED_KERNEL_NAME, "kernel_ms_avg": round(kern_ms, 4),
                     "kernel_ms_min": round(per[0], 4), "algorithmic_flops": flops, "algorithmic_bytes": io_bytes,
                     "hbm_frac_at_algorithmic_bytes": round(io_bytes / (kern_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
        "fwd_ms": round(kern_ms, 4),
        "pct_mfma_peak": round(100.0 * kern_tflops / MFMA_PEAK_TFLOPS, 2),
        "acsr_setup_ms": round(setup_ms, 2),
    }

    if not args.no_settle:
        # What limits the clock: power and clock while the headline kernel runs back to back, and the rate of the bare
        # matrix loop of the same tile shape (LDS reads + MFMAs only, random operands) under the same conditions.
        out["roofline"]["sustained"] = sample_power_and_clock(step)
        probe_data = torch.randn(32768, dtype=torch.float32).to(dtype).to(dev)
        if args.zero_operands:
            probe_data.zero_()
        import bench_probes as BP
        probe_tiles = 40
        loops = {}
        for shape, label in BP.PROBE_SHAPES.items():
            probe_wgs = B * H * (L // (256 if shape == 1 else 128))
            probe_out = torch.empty(probe_wgs * BP.PROBE_THREADS[shape], dtype=torch.float32, device=dev)
            probe = lambda s=shape, w=probe_wgs, o=probe_out: BP.check(BP.lib().splat_bench_mfma_lds_probe(
                probe_data.data_ptr(), probe_data.numel() * 2, o.data_ptr(), o.numel() * 4, s, w, probe_tiles, hip.stream_ptr(dev)),
                "splat_bench_mfma_lds_probe")
            settle(probe)
            probe_ms = min(time_batch(probe, 20, 5) for _ in range(3))
            probe_tflops = BP.lib().splat_bench_mfma_lds_probe_flops(shape, probe_wgs, probe_tiles) / (probe_ms * 1e-3) / 1e12
            loops[shape] = {"shape": label, "tflops": round(probe_tflops, 1), "frac_of_peak": round(probe_tflops / MFMA_PEAK_TFLOPS, 4),
                            "sustained": sample_power_and_clock(probe, 10)}
            del probe_out
        out["roofline"]["mfma_lds_loop"] = dict(
            loops[0], fused_frac_of_loop=round(kern_tflops / loops[0]["tflops"], 4),
            note="splat_bench_mfma_lds_probe shape 0: the fused kernel's LDS reads and MFMAs per tile and nothing else, N(0,1) "
                 "bf16 operands, same grid; its MFMAs are all counted, the fused figure counts nonzero FLOPs only",
            other_shapes=[loops[1], loops[2]])
        del probe_data

    extras = {}
    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if not args.no_extras:
        # the fused forward at the other four benchmark configurations, and on the reference's blocked mask
        # (acsr_helpers.py:18-34: every row block sees itself and the block before it) at config 4's shape with blocks
        # of 1024: 32 tiles per workgroup, none of them masked, against the 10 of the headline's band
        for name, (seed, Bc, Hc, Lc, dc, dt, pat, mul) in {
                "fused_cfg1": (1001, 1, 1, 512, 64, torch.float32, A.causal_windowed_pattern(512, 63), 1.0),
                "fused_cfg2": (1002, 4, 16, 4096, 64, torch.float16, A.causal_windowed_pattern(4096, 255), 0.5),
                "fused_cfg3": (1003, 2, 16, 8192, 64, torch.bfloat16, A.strided_patterns(8192, 128, 128), 1.0),
                "fused_cfg4": (1004, 2, 32, 8192, 128, torch.bfloat16, A.dilated_pattern(8192, 512, 2), 1.0),
                "fused_blocked_1024": (1006, 2, 32, 8192, 128, torch.bfloat16, A.blocked_pattern(8192, 1024), 1.0)}.items():
            qc, kc, vc = (t.mul(mul).to(dt).to(dev) for t in make_inputs(seed, Bc, Hc, Lc, dc, torch.float32))
            at = RegularAttention(Bc, Lc, Hc, dc, pat, 16, 16, dev, dt, scale=dc ** -0.5)
            nnz_c = sum(float(t[4].sum().item()) for t in at.segments.tuples)
            fl = 4.0 * dc * nnz_c * Bc * Hc
            byt = 4.0 * Bc * Hc * Lc * dc * qc.element_size()
            kTc = kc.transpose(2, 3)
            run = lambda: at([qc, kTc, vc])
            # (launches of 0.02-0.05 ms: the clock, which drops while the host builds the next case, needs some 40 ms of
            # them to come back: 0.051, 0.045, 0.043, 0.042, 0.041, 0.040 ms in six batches of 120 at config 2, then 0.0395)
            settle(run)
            ms = min(time_batch(run, 60, 60) for _ in range(3))
            peak = FP32_MFMA_PEAK_TFLOPS if dt == torch.float32 else MFMA_PEAK_TFLOPS
            extras[name] = {"ms": round(ms, 4), "tflops_nnz": round(fl / ms / 1e9, 2),
                            "pct_mfma_peak": round(100 * fl / ms / 1e9 / peak, 2),
                            "hbm_floor_ms": round(byt / HBM_PEAK_GBPS / 1e6, 4),
                            "pct_of_hbm_floor_rate": round(100 * byt / HBM_PEAK_GBPS / 1e6 / ms, 2)}
            # the reference's own layout of K: [B, H, d, L] contiguous (rows that step over columns cost a transpose of K)
            kTc = kTc.contiguous()
            settle(run)
            extras[name]["ms_kT_contiguous"] = round(min(time_batch(run, 60, 60) for _ in range(2)), 4)
            if name in ("fused_cfg2", "fused_cfg3"):
                # the fused backward at d = 64 (two launches: dQ, then dK and dV from one walk; config 3 adds the launch
                # that takes the transposed far field's 63 keys row by row), from the forward's output and row statistic
                xc = [qc, kc.transpose(2, 3), vc]
                oc, lc = at.forward_with_stats(xc)
                oc, lc = oc.clone(), lc.clone()
                gc = torch.randn_like(qc)
                at.backward_pass(xc, gc, lc, oc, fused=True)  # builds the transposed mask's ACSR and plan
                settle(lambda: at.backward_pass(xc, gc, lc, oc, fused=True))
                ms_b = min(time_batch(lambda: at.backward_pass(xc, gc, lc, oc, fused=True), 40, 20) for _ in range(3))
                extras["backward_" + name[6:]] = {"ms": round(ms_b, 4), "x_fused_forward": round(ms_b / ms, 2)}
                del xc, oc, lc, gc
            del at, qc, kc, vc, kTc
        # the d = 64 tile loop alone (both products out of LDS, one exponential per score, a barrier per tile: no loads, no
        # masks, no beginnings and ends of workgroups) in the kernel's wavefront shape and in thin wavefronts: what configs
        # 2 and 3 could reach if their workgroups had nothing but tiles to do
        import bench_probes as BP
        loop_data = (0.5 * torch.randn(32768, dtype=torch.float32)).to(torch.bfloat16).to(dev)
        loop_wgs, loop_tiles = 256 * 3 * 3, 64
        loop = {}
        for shape, label in BP.SOFTMAX_LOOP_SHAPES.items():
            loop_out = torch.empty(loop_wgs * BP.SOFTMAX_LOOP_THREADS[shape], dtype=torch.float32, device=dev)
            for with_exp in (1, 0):
                probe = lambda s=shape, e=with_exp, o=loop_out: BP.check(BP.lib().splat_bench_softmax_loop_probe(
                    loop_data.data_ptr(), loop_data.numel() * 2, o.data_ptr(), o.numel() * 4, s, e, loop_wgs, loop_tiles,
                    hip.stream_ptr(dev)), "splat_bench_softmax_loop_probe")
                settle(probe)
                ms_l = min(time_batch(probe, 20, 5) for _ in range(3))
                tf = BP.lib().splat_bench_softmax_loop_probe_flops(loop_wgs, loop_tiles) / (ms_l * 1e-3) / 1e12
                loop[("with" if with_exp else "without") + "_exponentials, " + label] = {
                    "workgroup_tiles_per_us": round(loop_wgs * loop_tiles / ms_l / 1e3, 1), "tflops": round(tf, 1),
                    "pct_mfma_peak": round(100 * tf / MFMA_PEAK_TFLOPS, 2)}
            del loop_out
        extras["tile_loop_d64"] = loop
        del loop_data
        # the literal reference layout: K^T contiguous [B, H, d, L]
        kT_c = kT_view.contiguous()
        _, per_c = time_launches(lambda: attn([qd, kT_c, vd]), max(5, args.steps // 2), max(3, args.warmup // 2))
        ms_c = sum(per_c) / len(per_c)
        extras["fused_kT_contiguous"] = {"ms": round(ms_c, 4), "tflops_nnz": round(flops / ms_c / 1e9, 2)}
        del kT_c

        # ACSR build on the config-5 mask (L*L bytes read once): create_acsr as a caller sees it (it ends with a read-back of
        # T, i.e. a stream synchronisation), and the builder's two kernels alone through the C ABI, each launch after a
        # 512 MiB write so that the freshly generated mask is not found in a cache
        mask = A.causal_windowed_pattern(L, w - 1).device_mask(dev)

        def build():
            A._MASK_CACHE.clear()
            A.create_acsr(mask, 16, dev)
        _, per_b = time_launches(build, 10, 2)
        ms_b = sum(per_b) / len(per_b)

        def build_known_T():   # the caller names the trailing dimension: nothing is read back, the call only enqueues
            A._MASK_CACHE.clear()
            A.create_acsr(mask, 16, dev, T=w)
        _, per_bt = time_launches(build_known_T, 10, 2)
        ms_bt = sum(per_bt) / len(per_bt)
        f32 = [torch.empty(L, dtype=torch.float32, device=dev) for _ in range(5)]
        spans = [torch.empty(-(-L // 16), dtype=torch.float32, device=dev) for _ in range(2)]
        ext = [torch.empty(L, dtype=torch.int32, device=dev) for _ in range(2)]
        summ = torch.empty(8, dtype=torch.int32, device=dev)
        flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)

        def build_kernels():
            rc = hip.lib().splat_acsr_build(mask.data_ptr(), L, L, mask.stride(0), 16, *[t.data_ptr() for t in f32 + spans + ext],
                                            summ.data_ptr(), hip.stream_ptr(dev))
            hip.check(rc, "splat_acsr_build")
        settle(build_kernels)
        _, per_k = time_launches(build_kernels, 10, 2)
        ms_k = sum(per_k) / len(per_k)
        ms_cold = time_cold_launches(build_kernels, flush, 10)
        extras["acsr_build_cfg5"] = {"ms_incl_readback": round(ms_b, 4), "ms_known_T": round(ms_bt, 4), "ms_kernels": round(ms_k, 4),
                                     "ms_kernels_caches_flushed": round(ms_cold, 4), "mask_bytes": L * L,
                                     "gbps_caches_flushed": round(L * L / ms_cold / 1e6, 1),
                                     "hbm_frac_caches_flushed": round(L * L / ms_cold / 1e6 / HBM_PEAK_GBPS, 4)}
        del mask, flush, f32, spans, ext, summ
        A._MASK_CACHE.clear()

        # unfused kernels at config 4 (dilated, B=2 H=32 L=8192 d=128 bf16, T=512): softmax GB/s is the metric's second half
        B4, H4, L4, d4 = 2, 32, 8192, 128
        q4, k4, v4 = make_inputs(1004, B4, H4, L4, d4, dtype)
        q4, k4, v4 = q4.to(dev), k4.to(dev), v4.to(dev)
        pat4 = A.dilated_pattern(L4, 512, 2)
        acsr = A.create_acsr(pat4, 16, dev)
        T4 = acsr[5]
        nnz4 = float(acsr[4].sum().item())
        s_buf = torch.empty(B4, H4, L4, T4, dtype=dtype, device=dev)
        p_buf = torch.empty_like(s_buf)
        o_buf = torch.empty(B4, H4, L4, d4, dtype=dtype, device=dev)
        k4T = k4.transpose(2, 3)
        run_sddmm = lambda: r_sddmm.rsddmm_launcher(q4, k4T, s_buf, acsr[0], acsr[1], acsr[2], acsr[3], T4, acsr[4], (1, 1),
                                                    None, None, 16, 16, scale=d4 ** -0.5)
        run_soft = lambda: r_softmax.rsoftmax_launcher(s_buf, p_buf, acsr[0], acsr[1], acsr[2], acsr[3], T4, 512, acsr[4],
                                                       (1, 1), 16)
        run_spmm = lambda: r_spmm.rspmm_launcher(p_buf, v4, o_buf, acsr[0], acsr[1], acsr[2], acsr[3], acsr[6], acsr[7],
                                                 T4, acsr[4], (1, 1, 1), 16, 16)
        # the product with the transposed compressed matrix (backward pass only; the reference has no counterpart)
        import r_backward
        segs4 = A.create_acsr_segments([pat4], 16, dev)
        segs4_t = r_backward.transposed_segments([pat4], 16, dev)
        run_spmm_t = lambda: r_backward.rspmm_t_launcher(p_buf, v4, o_buf, segs4, segs4_t)
        flush = torch.empty(512 << 20, dtype=torch.uint8, device=dev)  # > L2 + MALL: written before every "cold" launch
        for name, fn, byt, fl in (
                ("sddmm_cfg4", run_sddmm, (2 * B4 * H4 * L4 * d4 + nnz4 * B4 * H4) * 2, 2 * d4 * nnz4 * B4 * H4),
                ("softmax_cfg4", run_soft, 2 * nnz4 * B4 * H4 * 2, 0.0),
                ("spmm_cfg4", run_spmm, (2 * B4 * H4 * L4 * d4 + nnz4 * B4 * H4) * 2, 2 * d4 * nnz4 * B4 * H4),
                ("spmm_t_cfg4", run_spmm_t, (2 * B4 * H4 * L4 * d4 + nnz4 * B4 * H4) * 2, 2 * d4 * nnz4 * B4 * H4)):
            # back to back first (one event pair around all launches): these 150 launches are also what brings the clocks of
            # a GPU that has just been allocating and filling buffers up to where they stay; the per-launch figures that
            # follow are 10 % higher when taken first
            ms_b = min(time_batch(fn, 40, 10) for _ in range(3))
            _, pr = time_launches(fn, 40, 20)
            ms = sum(pr) / len(pr)
            extras[name] = {"ms": round(ms, 4), "ms_caches_flushed": round(time_cold_launches(fn, flush, 20), 4),
                            "ms_back_to_back": round(ms_b, 4),
                            "gbps_algorithmic": round(byt / ms / 1e6, 1),
                            "gbps_back_to_back": round(byt / ms_b / 1e6, 1),
                            "hbm_frac": round(byt / ms / 1e6 / HBM_PEAK_GBPS, 4)}
            if fl:
                extras[name]["tflops_nnz"] = round(fl / ms / 1e9, 2)
        out["softmax_gbps"] = extras["softmax_cfg4"]["gbps_algorithmic"]
        # the read + write streaming ceiling: a plain 1 GiB copy by a kernel of this library with the softmax's access forms
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        import bench_probes as BP
        copy = lambda: BP.check(BP.lib().splat_bench_stream_copy(src.data_ptr(), dst.data_ptr(), src.numel(), hip.stream_ptr(dev)),
                                "splat_bench_stream_copy")
        ms = min(time_batch(copy, 10, 3) for _ in range(3))
        extras["stream_copy_1GiB"] = {"ms": round(ms, 4), "gbps_read_plus_write": round(2 * src.numel() / ms / 1e6, 1)}
        # both sides timed the same way: back-to-back launches
        extras["softmax_cfg4"]["frac_of_stream_copy"] = round(extras["softmax_cfg4"]["gbps_back_to_back"] /
                                                              extras["stream_copy_1GiB"]["gbps_read_plus_write"], 4)
        del src, dst
        # the softmax on config 3's compressed rows: two segments, T = 191 slots, so rows begin anywhere inside a 16-byte chunk
        pat3 = A.strided_patterns(8192, 128, 128)
        segs3 = A.create_acsr_segments(pat3, 16, dev)
        B3, H3, L3, T3 = 2, 16, 8192, segs3.T
        live3 = int(sum(float(t[4].sum()) for t in segs3.tuples))
        s3 = torch.randn(B3, H3, L3, T3, device=dev, dtype=dtype)
        p3 = torch.empty_like(s3)
        sg0 = segs3.tuples[0]
        run_soft3 = lambda: r_softmax.rsoftmax_launcher(s3, p3, sg0[0], sg0[1], sg0[2], sg0[3], T3, 256, sg0[4], (1, 1), 16, segments=segs3)
        settle(run_soft3)
        ms = min(time_batch(run_soft3, 40, 10) for _ in range(3))
        byt3 = 2 * live3 * B3 * H3 * 2
        extras["softmax_cfg3"] = {"ms": round(ms, 4), "T": T3, "gbps_algorithmic": round(byt3 / ms / 1e6, 1),
                                  "hbm_frac": round(byt3 / ms / 1e6 / HBM_PEAK_GBPS, 4)}
        del s3, p3
        del s_buf, p_buf, o_buf, flush
        # backward pass (not in the reference) at the same shape: nonzero FLOPs = 2.5 x the forward's (five products).  The
        # fused kernel takes the forward's output and row statistic; the composed pass (operators over compressed matrices)
        # is timed with and without the statistic.
        attn4 = RegularAttention(B4, L4, H4, d4, pat4, 16, 16, dev, dtype, scale=d4 ** -0.5)
        g4 = torch.randn_like(q4)
        x4 = [q4, k4T, v4]
        out4, lse4 = attn4.forward_with_stats(x4)
        out4, lse4 = out4.clone(), lse4.clone()
        fl4 = 10 * d4 * nnz4 * B4 * H4
        ms_f = min(time_batch(lambda: attn4.backward_pass(x4, g4, lse4, out4, fused=True), 10, 3) for _ in range(3))
        _, pr = time_launches(lambda: attn4.backward_pass(x4, g4, lse4, fused=False), 10, 3)
        ms_c = sum(pr) / len(pr)
        _, pr = time_launches(lambda: attn4.backward_pass(x4, g4, fused=False), 10, 3)
        ms_c0 = sum(pr) / len(pr)
        extras["backward_cfg4"] = {"ms": round(ms_f, 4), "tflops_nnz": round(fl4 / ms_f / 1e9, 2),
                                   "x_fused_forward": round(ms_f / extras["fused_cfg4"]["ms"], 2),
                                   "kernel": "splat_attention_bwd: three launches of attn_bwd_kernel at d = 128 (dQ, which also computes the row sums of dO * O; dK; dV), no compressed matrix",
                                   "composed_ms_with_forward_lse": round(ms_c, 3), "composed_ms": round(ms_c0, 3)}
        del out4, lse4
        del attn4, g4, q4, k4, v4
        # the fused backward at the headline shape (config 5), from the forward's output and row statistic
        g5 = torch.randn_like(qd)
        x5 = [qd, kT_view, vd]
        out5, lse5 = attn.forward_with_stats(x5)
        out5, lse5 = out5.clone(), lse5.clone()
        attn.backward_pass(x5, g5, lse5, out5, fused=True)  # builds the transposed mask's ACSR and plan
        ms_b5 = min(time_batch(lambda: attn.backward_pass(x5, g5, lse5, out5, fused=True), 10, 3) for _ in range(3))
        extras["backward_cfg5"] = {"ms": round(ms_b5, 4), "tflops_nnz": round(2.5 * flops / ms_b5 / 1e9, 2),
                                   "x_fused_forward": round(ms_b5 / kern_ms, 2)}
        del g5, out5, lse5
    out["extras"] = extras

    if not args.no_cpu:
        # the reference's dense masked path (einsum of r_sddmm.py:186-188, masked softmax, matmul) in fp32 on the
        # host cores, on `cpu_heads` (batch, head) pairs of the same workload; nonzero FLOPs counted as above
        n = max(1, args.cpu_heads)
        ii = np.arange(L)
        mask_rows = lambda a, c: (ii[a:c, None] >= ii[None, :]) & (ii[a:c, None] - (w - 1) <= ii[None, :])
        qs, ks, vs = q.reshape(B * H, 1, L, d)[:n], k.reshape(B * H, 1, L, d)[:n], v.reshape(B * H, 1, L, d)[:n]
        from oracle import splat_oracle as O  # the checker and CPU baseline; nothing above this line touches it
        t0 = time.perf_counter()
        ref = O.dense_masked_attention_chunked(qs.transpose(0, 1), ks.transpose(0, 1).transpose(2, 3), vs.transpose(0, 1),
                                               mask_rows, scale)
        cpu_s = time.perf_counter() - t0
        got = attn([qd, kT_view, vd]).float().reshape(B * H, L, d)[:n].cpu()
        err = float((got - ref[0]).abs().max())
        out["cpu_baseline"] = {"value": round(4.0 * d * nnz * n / cpu_s / 1e12, 5), "unit": out["unit"],
                               "cores": torch.get_num_threads(), "kind": "port",
                               "sample": f"{n} of {B * H} (batch, head) pairs of config 5, dense fp32 masked attention "
                                         f"in PyTorch on the host, {cpu_s:.1f} s",
                               "max_abs_err_gpu_vs_cpu": round(err, 5)}

    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
