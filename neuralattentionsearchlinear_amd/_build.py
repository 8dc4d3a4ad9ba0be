"""Builds csrc/*.hip into csrc/libnatsl.so for gfx950 with hipcc (cross-compiles without a GPU), and the benchmark's
clock probe (csrc/bench/) into csrc/libnatsl_bench.so, which is not part of the C ABI."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB = os.path.join(CSRC, "libnatsl.so")
BENCH_LIB = os.path.join(CSRC, "libnatsl_bench.so")
SOURCES = ["natsl_route.hip", "natsl_softmax.hip", "natsl_softmax_bwd.hip", "natsl_linear.hip", "natsl_linear_bwd.hip", "natsl_norm_gate.hip", "natsl_conv.hip", "natsl_decode.hip", "natsl_cache.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # keep the compiler from forming packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    *os.environ.get("NATSL_HIPCC_EXTRA", "").split(),  # extra compiler flags for a development build
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False) -> str:
    hipcc = _hipcc()
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = []

    def compile_one(src):
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
        if verbose and r.stderr.strip():
            print(r.stderr, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(4, len(srcs))) as ex:
        objs = list(ex.map(compile_one, srcs))
    r = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    r = subprocess.run([hipcc, *FLAGS, "-shared", os.path.join(CSRC, "bench", "bench_probe.hip"), "-o", BENCH_LIB], capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on bench/bench_probe.hip:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
