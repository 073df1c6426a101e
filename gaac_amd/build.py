"""Builds gaac_amd/libgaac_hip.so (hand-written HIP kernels for gfx950 + the extern "C" entry points) with hipcc.

    python -m gaac_amd.build          # or: from gaac_amd.build import build; build()

The library is built in-tree; nothing is compiled at import time or on the GPU box."""
from __future__ import annotations
import os, subprocess, sys, shutil

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libgaac_hip.so")
LIB_W12 = os.path.join(HERE, "libgaac_hip_w12.so")            # measurement build -DGAAC_WAVES12: twelve-wave blocks, three waves per SIMD (see attn.hip); on demand only
LIB_TIMING = os.path.join(HERE, "libgaac_hip_timing.so")      # same sources with -DGAAC_PHASE_TIMING (per-block phase time stamps); built on demand only
SOURCES = ["codec.hip", "attn.hip", "cache.hip", "paged.hip"]
# bench.py's measurement aids (read probe, plain copy): their own library next to bench.py, not in the product library
BENCH_SRC = os.path.join(os.path.dirname(HERE), "bench_kernels.hip")
BENCH_LIB = os.path.join(os.path.dirname(HERE), "libgaac_bench.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", 
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",      # never emit packed-FP32 VALU ops
         # atomics here are issued by one chosen lane (the tile counter in LDS): skip the compiler's wave-wide aggregation code
         "-mllvm", "-amdgpu-atomic-optimizer-strategy=None",
         "-Wno-unused-command-line-argument"]
# per source: the attention kernels' tile loop is a long chain of dependent LDS look-ups, decode arithmetic and matrix products with
# only two waves per SIMD to hide latencies behind; the scheduler's ILP-first strategy measured 0.3 us faster per launch on config 1
SOURCE_FLAGS = {"attn.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"]}


def build(verbose: bool = True, extra_flags: list[str] | None = None, timing: bool = False, waves12: bool = False) -> str:
    """timing=True builds the instrumented variant (libgaac_hip_timing.so), waves12=True the twelve-wave measurement build
    (libgaac_hip_w12.so); both are loaded through the GAAC_HIP_LIB override and neither is part of the product."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objs = []
    if timing: extra_flags = [*(extra_flags or []), "-DGAAC_PHASE_TIMING"]
    if waves12: extra_flags = [*(extra_flags or []), "-DGAAC_WAVES12"]
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".timing.o" if timing else ".w12.o" if waves12 else ".o"))
        cmd = [hipcc, *FLAGS, *SOURCE_FLAGS.get(src, []), *(extra_flags or []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose: print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip(): print(err, file=sys.stderr)
        objs.append(obj)
    out = LIB_TIMING if timing else LIB_W12 if waves12 else LIB
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", out]
    if verbose: print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return out


def build_bench_lib(verbose: bool = True) -> str:
    """bench_kernels.hip -> libgaac_bench.so (beside bench.py)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    cmd = [hipcc, *FLAGS, "-I", CSRC, "-shared", BENCH_SRC, "-o", BENCH_LIB]
    if verbose: print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on bench_kernels.hip:\n" + "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l))
    return BENCH_LIB


if __name__ == "__main__":      # no option: the library and bench.py's kernels; --timing / --waves12: only that measurement build
    if "--timing" in sys.argv: print(build(timing=True))
    if "--waves12" in sys.argv: print(build(waves12=True))
    if "--timing" not in sys.argv and "--waves12" not in sys.argv:
        print(build())
        print(build_bench_lib())
