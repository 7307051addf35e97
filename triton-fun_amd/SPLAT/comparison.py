"""Sparse kernels against dense ones over a sweep of the sparsity parameter.

Successor of the reference's ``SPLAT/comparison.py`` (:76-106): the same sweep, the sparsity parameter doubling from 2
up to the sequence length for the "Blocked" and "Windowed" patterns, with the baselines available on this platform
instead of Triton's block-sparse matmul (``triton.ops`` no longer exists): the dense product the reference's own
``truth`` uses (``r_sddmm.py:186-188``) for the SDDMM, and ``torch.nn.functional.scaled_dot_product_attention`` with a
boolean mask for the fused forward.  Nothing runs at import; ``python comparison.py`` prints both sweeps.
"""
from __future__ import annotations

from typing import Any, Callable

import torch

import _splat_hip as _hip
from acsr_helpers import blocked_pattern, create_acsr, windowed_pattern
from r_attention import RegularAttention
from r_sddmm import rsddmm_launcher, rsddmm_preamble

_PATTERNS = {"Blocked": blocked_pattern, "Windowed": windowed_pattern}


def _time_ms(fn: Callable[[], Any], iters: int = 20, warmup: int = 5) -> float:
    for _ in range(warmup):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / iters


def _pattern(pattern: str, sequence_length: int, sparsity_parameter: int):
    if pattern not in _PATTERNS:
        raise Exception("Not implemented!")  # the reference's message, comparison.py:104
    return _PATTERNS[pattern](sequence_length, sparsity_parameter)


def benchmark(pattern: str, sequence_length: int, BLOCK_SIZE_Y: int, BLOCK_SIZE_X: int, GPU_ID: Any,
              verbose: bool = True, *, batch: int = 1, num_heads: int = 1, inner_dim: int | None = None,
              dtype: torch.dtype = torch.float32) -> list[dict]:
    """The reference's SDDMM sweep: left [.., sequence_length, inner_dim] and right [.., inner_dim, sequence_length]
    matrices of small integers (the reference: one float32 pair with inner_dim = sequence_length, which keeps 8 of this
    GPU's 256 compute units busy; ``batch`` / ``num_heads`` / ``inner_dim`` / ``dtype`` give it a realistic shape), one
    launch of the compressed SDDMM against the dense product of the same operands.  Returns one record per sparsity
    parameter: {'sparsity_parameter', 'nnz', 'splat_ms', 'dense_ms'} (nnz per (batch, head))."""
    dev = _hip.resolve_device(GPU_ID)
    inner = sequence_length if inner_dim is None else inner_dim
    rows = []
    sparsity_parameter = 2
    while sparsity_parameter <= sequence_length:
        g = torch.Generator().manual_seed(sparsity_parameter)
        left = torch.randint(0, 100, (batch, num_heads, sequence_length, inner), generator=g).to(dtype).to(dev)
        right = torch.randint(0, 100, (batch, num_heads, inner, sequence_length), generator=g).to(dtype).to(dev)
        mask = _pattern(pattern, sequence_length, sparsity_parameter)
        meta = create_acsr(mask, BLOCK_SIZE_Y, GPU_ID)
        T = meta[5]
        out, grid, tbx, tby = rsddmm_preamble(mask, (batch, num_heads, sequence_length, T), BLOCK_SIZE_X, BLOCK_SIZE_Y,
                                              GPU_ID, dtype)
        splat = _time_ms(lambda: rsddmm_launcher(left, right, out, meta[0], meta[1], meta[2], meta[3], T, meta[4], grid,
                                                 tbx, tby, BLOCK_SIZE_Y, BLOCK_SIZE_X))
        dense = _time_ms(lambda: torch.einsum("bnqd,bndk->bnqk", left, right))
        rows.append({"sparsity_parameter": sparsity_parameter, "nnz": int(meta[4].sum().item()),
                     "splat_ms": splat, "dense_ms": dense})
        if verbose:
            print(f"sparsity parameter: {sparsity_parameter:5d}  nnz {rows[-1]['nnz']:8d}  "
                  f"SPLAT sddmm {splat:.4f} ms  dense {dense:.4f} ms", flush=True)
        sparsity_parameter *= 2
    return rows


def benchmark_attention(pattern: str, sequence_length: int, GPU_ID: Any, batch: int = 4, num_heads: int = 16,
                        head_dim: int = 128, dtype: torch.dtype = torch.bfloat16, verbose: bool = True) -> list[dict]:
    """The same sweep for the whole forward: ``RegularAttention`` (fused kernel) against PyTorch's scaled-dot-product
    attention given the same mask as a boolean tensor.  Records: {'sparsity_parameter', 'splat_ms', 'dense_ms',
    'max_abs_diff'}."""
    dev = _hip.resolve_device(GPU_ID)
    g = torch.Generator().manual_seed(sequence_length)
    q, k, v = [torch.randn(batch, num_heads, sequence_length, head_dim, generator=g).to(dtype).to(dev) for _ in range(3)]
    scale = head_dim ** -0.5
    rows = []
    sparsity_parameter = 2
    while sparsity_parameter <= sequence_length:
        mask = _pattern(pattern, sequence_length, sparsity_parameter)
        attn = RegularAttention(batch, sequence_length, num_heads, head_dim, mask, 16, 16, GPU_ID, dtype, scale=scale)
        allowed = mask.device_mask(dev).bool()
        kT = k.transpose(2, 3)
        splat = _time_ms(lambda: attn([q, kT, v]))
        sdpa = lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=allowed, scale=scale)  # noqa: E731
        dense = _time_ms(sdpa)
        diff = float((attn([q, kT, v]).float() - sdpa().float()).abs().max())
        rows.append({"sparsity_parameter": sparsity_parameter, "splat_ms": splat, "dense_ms": dense, "max_abs_diff": diff})
        if verbose:
            print(f"sparsity parameter: {sparsity_parameter:5d}  SPLAT fused {splat:.4f} ms  dense SDPA {dense:.4f} ms  "
                  f"({dense / splat:5.1f}x)  max |diff| {diff:.3g}", flush=True)
        sparsity_parameter *= 2
    return rows


if __name__ == "__main__":
    sequence_length: int = 1024   # the reference's settings, comparison.py:108-112
    BLOCK_SIZE_X: int = 16
    BLOCK_SIZE_Y: int = 16
    GPU_ID: int = 0
    for pattern in ("Windowed", "Blocked"):
        print(f"-- SDDMM, {pattern}, sequence length {sequence_length}")
        benchmark(pattern, sequence_length, BLOCK_SIZE_Y, BLOCK_SIZE_X, GPU_ID)
    print("-- SDDMM, Windowed, B=4 H=16 L=4096 d=128 bf16")
    benchmark("Windowed", 4096, BLOCK_SIZE_Y, BLOCK_SIZE_X, GPU_ID, batch=4, num_heads=16, inner_dim=128, dtype=torch.bfloat16)
    for pattern in ("Windowed", "Blocked"):
        print(f"-- fused forward, {pattern}, B=4 H=16 L=4096 d=128 bf16")
        benchmark_attention(pattern, 4096, GPU_ID)
