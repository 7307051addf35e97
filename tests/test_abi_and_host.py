"""No-GPU checks of the product: the C-ABI library loads and exports every symbol the header declares,
rejects bad arguments before touching the device, and the Python operator layer refuses to run
without a HIP device (there is no host fallback)."""
import ctypes
import os
import re

import pytest
import torch

import _splat_hip as hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "splat_hip.h")


def header_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(splat_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    syms = header_symbols()
    assert {"splat_acsr_build", "splat_mask_generate", "splat_sddmm", "splat_softmax", "splat_spmm",
            "splat_attention_fwd", "splat_attention_plan_bytes", "splat_attention_plan", "splat_attention_fwd_planned", "splat_attention_fwd_stats", "splat_sddmm_probs",
            "splat_version", "splat_last_error"} <= set(syms)
    handle = ctypes.CDLL(hip.LIB_PATH)
    for s in syms:
        assert hasattr(handle, s), s
    assert sorted(hip.EXPORTS) == syms


def test_the_measurement_library_exports_what_its_header_declares():
    """libsplat_bench.so (bench.py's two ceilings) against include/splat_bench.h and its binding; and the operator header
    declares none of it."""
    import bench_probes as BP
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "splat_bench.h")).read(), flags=re.S)
    syms = sorted(set(re.findall(r"\b(splat_bench_[a-z_0-9]+)\s*\(", text)))
    assert "splat_bench_stream_copy" in syms and "splat_bench_mfma_lds_probe" in syms
    handle = ctypes.CDLL(BP.LIB_PATH)
    for s in syms:
        assert hasattr(handle, s), s
    assert sorted(BP.EXPORTS) == syms
    want = int(re.search(r"#define SPLAT_BENCH_VERSION (\d+)", open(os.path.join(ROOT, "include", "splat_bench.h")).read()).group(1))
    assert BP.lib().splat_bench_version() == want
    assert not [s for s in header_symbols() if "probe" in s or "stream_copy" in s or "bench" in s]
    assert BP.lib().splat_bench_stream_copy(None, None, 16, None) == -1 and b"null" in BP.lib().splat_bench_last_error()


def test_version_matches_header():
    want = int(re.search(r"#define SPLAT_VERSION (\d+)", open(HEADER).read()).group(1))
    assert hip.lib().splat_version() == want


def test_null_and_shape_arguments_are_rejected_without_a_device():
    lib = hip.lib()
    assert lib.splat_softmax(None, None, None, 1, 1, 1, 1, 0, 0, None) == -1
    assert b"null" in lib.splat_last_error()
    seg = (hip.AcsrSeg * 1)()
    assert lib.splat_softmax(8, 8, seg, 0, 1, 1, 1, 0, 0, None) == -2          # n_seg = 0
    assert lib.splat_softmax(8, 8, seg, 1, 1, 1, 0, 0, 0, None) == -2          # T = 0
    assert lib.splat_acsr_build(None, 4, 4, 4, 2, *([None] * 10), None) == -1
    assert lib.splat_acsr_build(8, 4, 4, 2, 2, *([8] * 7), None, None, 8, None) == -2  # ld < cols
    assert lib.splat_mask_generate(8, 4, 4, 4, 99, 1, 1, None) == -5
    assert lib.splat_attention_fwd(8, 0, 0, 64, 8, 0, 0, 1, 64, 8, 0, 0, 64, 8, 0, 0, 64, seg, 1, 1, 1, 16, 48, 1.0, 2,
                                   None) == -5                                   # d = 48 unsupported
    assert b"64 or 128" in lib.splat_last_error()
    assert lib.splat_attention_fwd_planned(8, 0, 0, 64, 8, 0, 0, 1, 64, 8, 0, 0, 64, 8, 0, 0, 64, seg, 1, 1, 1, 16, 48, 1.0, 2,
                                           16, 1 << 20, None) == -5
    assert b"splat_attention_fwd_planned" in lib.splat_last_error()
    assert lib.splat_sddmm(8, 0, 0, 8, 8, 0, 0, 3, 5, 8, seg, 1, 1, 1, 4, 4, 8, 4, 1.0, 0, 0, None) == -4  # no unit stride
    assert lib.splat_spmm(8, 8, 0, 0, 8, 8, seg, 1, 1, 1, 4, 4, 8, 4, 7, 0, None) == -3                    # bad dtype


def test_the_allocation_free_forward_rejects_what_its_built_in_buffer_cannot_hold():
    lib = hip.lib()
    seg = (hip.AcsrSeg * 2)()
    for i in range(2):
        seg[i].sTod_lin = seg[i].sTod_trans = seg[i].nnz = 8
        seg[i].row_stride_hint = 1
    fwd = lambda n_seg, L: lib.splat_attention_fwd_noalloc(8, 0, 0, 64, 8, 0, 0, 1, 64, 8, 0, 0, 64, 8, 0, 0, 64, seg, n_seg, 1, 1, L,
                                                           64, 1.0, 2, None)
    L_big = 1 << 18
    assert lib.splat_attention_plan_bytes(seg, 1, L_big) > hip.STATIC_PLAN_BYTES
    assert fwd(1, L_big) == -2
    msg = lib.splat_last_error()
    assert b"splat_attention_fwd_noalloc" in msg and b"built-in buffer" in msg and str(hip.STATIC_PLAN_BYTES).encode() in msg
    assert fwd(0, 128) == -2 and fwd(1, 0) == -2
    assert lib.splat_attention_fwd_noalloc(8, 0, 0, 64, 8, 0, 0, 1, 64, 8, 0, 0, 64, 8, 0, 0, 64, None, 1, 1, 1, 128, 64, 1.0, 2,
                                           None) == -1
    header = open(HEADER).read()
    assert int(eval(re.search(r"#define SPLAT_STATIC_PLAN_BYTES \((.*?)\)", header).group(1))) == hip.STATIC_PLAN_BYTES


def test_the_fused_backward_checks_its_arguments_on_the_host():
    """splat_attention_bwd refuses what its kernel is not built for before anything is launched."""
    lib = hip.lib()
    seg = (hip.AcsrSeg * 1)()
    seg[0].sTod_lin = seg[0].sTod_trans = seg[0].nnz = 16
    seg[0].row_stride_hint = 1
    L, d = 256, 64
    need = lib.splat_attention_plan_bytes(seg, 1, L)

    def bwd(q=16, lse=16, d=d, dtype=2, scale=1.0, plan_bytes=need, q_sl=d, seg_t=seg):
        t = [16, 0, 0, d]  # pointer, batch / head / row strides
        return lib.splat_attention_bwd(q, 0, 0, q_sl, *t, *t, *t, *t, lse, 16, 16, 16, 16, seg, 1, 16, plan_bytes,
                                       seg_t, 1, 16, need, 1, 1, L, d, scale, dtype, None)
    assert bwd(q=None) == -1 and bwd(lse=None) == -1 and bwd(seg_t=None) == -1
    assert bwd(d=96) == -5 and b"64 or 128" in lib.splat_last_error()
    assert bwd(dtype=0) == -5 and b"16-bit" in lib.splat_last_error()
    assert bwd(scale=0.0) == -5
    assert bwd(q=24) == -4 and bwd(q_sl=d + 4) == -4
    assert bwd(q_sl=32) == -2
    assert bwd(plan_bytes=need - 16) == -2 and b"plan" in lib.splat_last_error()


def test_the_key_transpose_checks_its_arguments_on_the_host():
    lib = hip.lib()

    def tr(src=16, dst=16, L=100, d=64, sd=100, dtype=2):
        return lib.splat_transpose_keys(src, 0, 0, sd, dst, 1, 1, L, d, dtype, None)
    assert tr(src=None) == -1 and tr(dst=None) == -1
    assert tr(L=0) == -2 and tr(d=0) == -2
    assert tr(sd=99) == -2 and b"stride" in lib.splat_last_error()
    assert tr(dtype=7) == -3
    assert tr(dst=24) == -4 and tr(src=17) == -4


def test_plan_size_is_host_arithmetic():
    lib = hip.lib()
    seg = (hip.AcsrSeg * 2)()
    # per variant and segment: per 128-row block one plan record, four wavefront spans and 128 row windows of 16 bytes
    assert lib.splat_attention_plan_bytes(seg, 1, 16384) == 2 * 128 * (5 + 128) * 16
    assert lib.splat_attention_plan_bytes(seg, 2, 130) == 2 * 2 * 2 * (5 + 128) * 16
    seg[0].row_stride_hint = seg[1].row_stride_hint = 2        # rows 0, 2, 4, .. and 1, 3, 5, .. in separate blocks
    assert lib.splat_attention_plan_bytes(seg, 2, 130) == 2 * 2 * 2 * (5 + 128) * 16
    assert lib.splat_attention_plan_bytes(seg, 2, 300) == 2 * 2 * 4 * (5 + 128) * 16
    assert lib.splat_attention_plan_bytes(seg, 0, 16) == 0 and lib.splat_attention_plan_bytes(None, 1, 16) == 0
    assert lib.splat_attention_plan(seg, 1, 16, None, 0, None) == -1
    seg[0].sTod_lin = seg[0].sTod_trans = seg[0].nnz = 8
    assert lib.splat_attention_plan(seg, 1, 16, 16, 100, None) == -2 and b"bytes" in lib.splat_last_error()
    assert lib.splat_attention_plan(seg, 1, 16, 24, 1 << 20, None) == -4      # misaligned plan


def test_operators_refuse_the_host():
    import acsr_helpers as A
    import r_attention
    with pytest.raises(hip.SplatError):
        A.create_acsr(A.create_blocked_mask(10, 2), 2, "cpu")
    with pytest.raises(hip.SplatError):
        r_attention.RegularAttention(1, 16, 1, 64, A.create_causal_windowed_mask(16, 3), 16, 16, "cpu", torch.float32)
    if not torch.cuda.is_available():
        with pytest.raises(hip.SplatError):
            A.create_acsr(A.create_blocked_mask(10, 2), 2, 0)


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "triton-fun_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text, os.path.join(base, f)
