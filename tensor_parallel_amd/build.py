"""Builds `tensor_parallel_amd/_lib/libtpamd.so` (the C ABI of include/tpamd.h) with hipcc for gfx950.

Run `python -m tensor_parallel_amd.build`. hipcc cross-compiles, so no GPU is needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OUT_DIR = PKG / "_lib"
LIB = OUT_DIR / "libtpamd.so"
SOURCES = ["api.hip", "runtime.hip", "noalloc.hip", "slice.hip", "reduce.hip", "gemm.hip", "skinny.hip", "attention.hip", "rope.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU ops are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _compile(src: str, verbose: bool) -> Path:
    obj = OUT_DIR / (src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so on every file: drop that line
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in res.stderr.splitlines() if noise not in line)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = True, jobs: int = 4) -> Path:
    """Compile every HIP source and link the shared library. Always recompiles."""
    OUT_DIR.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs), "-Wl,-soname,libtpamd.so"]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB


if __name__ == "__main__":
    print(build())
