"""Builds libovfcc.so (C ABI + HIP kernels for gfx950) and libovfcc_bench.so (the benchmark's timing helpers and
probe kernels, linked against the former) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libovfcc.so")
BENCH_LIB = os.path.join(PKG, "libovfcc_bench.so")
SOURCES = ["api.cpp", "repack.cpp", "plan.cpp", "fold.cpp", "fold_data.cpp", "kernel_plain.hip", "scratch.hip", "kernel_decode.hip", "kernel_gemv.hip", "kernel_gemv16.hip", "kernel_gemv16s.hip", "kernel_mlp.hip", "kernel_batch.hip", "kernel_prefill.hip", "kernel_prefill_direct.hip", "kernel_prefill_async.hip", "kernel_prefill_big.hip",
           "kernel_prefill_wide.hip", "kernel_prefill_i8.hip", "kernel_prefill_i8w4.hip"]
BENCH_SOURCES = ["bench.cpp", "bench_probe.hip"]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def _hipcc(sources, out, extra, verbose):
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-pthread",
           # keep the compiler from forming packed-FP32 instructions
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    cmd += [os.path.join(CSRC, s) for s in sources]
    cmd += extra + ["-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed building " + os.path.basename(out))


def build_library(verbose: bool = False) -> str:
    _hipcc(SOURCES, LIB, [], verbose)
    # the benchmark library finds the product library beside itself
    _hipcc(BENCH_SOURCES, BENCH_LIB, ["-L" + PKG, "-lovfcc", "-Wl,-rpath,$ORIGIN"], verbose)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
