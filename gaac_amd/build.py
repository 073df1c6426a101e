"""Builds gaac_amd/libgaac_hip.so (hand-written HIP kernels for gfx950 + the extern "C" entry points) with hipcc.

    python -m gaac_amd.build          # or: from gaac_amd.build import build; build()

The library is built in-tree; nothing is compiled at import time or on the GPU box."""
from __future__ import annotations
import os, subprocess, sys, shutil

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libgaac_hip.so")
SOURCES = ["codec.hip", "attn.hip", "cache.hip", "paged.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", 
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",      # never emit packed-FP32 VALU ops
         "-Wno-unused-command-line-argument"]


def build(verbose: bool = True, extra_flags: list[str] | None = None) -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *(extra_flags or []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose: print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{err}")
        if verbose and err.strip(): print(err, file=sys.stderr)
        objs.append(obj)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    if verbose: print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
