#!/usr/bin/env python3
"""Compile the HIP sources under csrc/ into mase_hip/lib/libmase_hip.so for gfx950.

    python mase-triton_amd/build.py [--force] [--save-temps]

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
from __future__ import annotations

import argparse
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
OBJ = os.path.join(ROOT, "build")
LIB_DIR = os.path.join(ROOT, "mase_hip", "lib")
LIB = os.path.join(LIB_DIR, "libmase_hip.so")
# helpers of the benchmark and the tests (a tuned streaming copy as yardstick; the SwiGLU arithmetic on its own); not part of
# the product's C ABI
BENCH_SRCS = [os.path.join(CSRC, "bench", f) for f in ("stream_copy.hip", "swiglu_probe.hip")]
BENCH_LIB = os.path.join(LIB_DIR, "libmase_bench.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _includes(path: str, seen: set[str] | None = None) -> set[str]:
    """The files `path` includes with quotes, transitively (what its object file depends on besides itself)."""
    seen = set() if seen is None else seen
    with open(path) as f:
        for m in re.finditer(r'^\s*#\s*include\s+"([^"]+)"', f.read(), re.M):
            inc = os.path.normpath(os.path.join(os.path.dirname(path), m.group(1)))
            if inc not in seen and os.path.exists(inc):
                seen.add(inc)
                _includes(inc, seen)
    return seen


def _stale(target: str, deps: list[str]) -> bool:
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build_library(force: bool = False, save_temps: bool = False, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def compile_one(pair):
        src, obj = pair
        if not (force or _stale(obj, [src, *_includes(src)])):
            return
        cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
        if save_temps:
            cmd += ["-save-temps=obj"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True, cwd=OBJ)

    with ThreadPoolExecutor(max_workers=min(7, len(srcs))) as ex:
        list(ex.map(compile_one, zip(srcs, objs)))
    if force or _stale(LIB, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    if force or _stale(BENCH_LIB, BENCH_SRCS + [h for src in BENCH_SRCS for h in _includes(src)]):
        cmd = [HIPCC, *FLAGS, "-shared", *BENCH_SRCS, "-o", BENCH_LIB]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True)
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--save-temps", action="store_true")
    a = ap.parse_args()
    print(build_library(force=a.force, save_temps=a.save_temps))
