"""Build libsplat_hip.so (the operators) and libsplat_bench.so (bench.py's measurement aids) for gfx950 from csrc/ with
hipcc.  Usage: python build.py [-j N]"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libsplat_hip.so")
BENCH_LIB = os.path.join(LIB_DIR, "libsplat_bench.so")

SOURCES = ["api_common.cpp", "acsr_build.hip", "softmax.hip", "sddmm.hip", "sddmm_lines.hip", "spmm.hip", "spmm_thin.hip", "spmm_tile.hip", "spmm_t_thin.hip", "attention.hip", "backward.hip", "attention_bwd.hip", "transpose.hip"]
# the measurement aids: a library of their own, so that the operator ABI holds operators only
BENCH_SOURCES = ["api_common.cpp", "bench_probes.hip"]
# packed fp32 VALU forms are switched off for every device compile
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function", "-Wno-inline-asm",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src: str) -> str:
    obj = os.path.join(OBJ, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
    noise = [l for l in r.stderr.splitlines() if l.strip() and "packed-fp32-ops" not in l]
    if noise:
        sys.stderr.write("\n".join(noise) + "\n")
    return obj


def _link(lib: str, objs: list[str]) -> None:
    # -Bsymbolic: each library calls its own copy of the shared helpers, whatever else the process has loaded
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", lib, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    # a kernel stub the host pass failed to emit only shows up when the library is loaded: check here
    undefined = subprocess.run(["nm", "-D", "--undefined-only", lib], capture_output=True, text=True).stdout
    missing = [l.split()[-1] for l in undefined.splitlines() if "splat" in l]
    if missing:
        raise RuntimeError(f"{lib} has undefined symbols of its own: {missing[:4]}")


def build(jobs: int = 8, verbose: bool = True) -> str:
    """Compile every source and link both shared libraries; always recompiles."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    names = SOURCES + [s for s in BENCH_SOURCES if s not in SOURCES]
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, 16))) as ex:
        objs = dict(zip(names, ex.map(_compile, names)))
    _link(LIB, [objs[s] for s in SOURCES])
    _link(BENCH_LIB, [objs[s] for s in BENCH_SOURCES])
    if verbose:
        print(f"built {LIB} and {BENCH_LIB}")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("-j", type=int, default=8)
    a = ap.parse_args()
    build(a.j)
