"""Builds dax_amd/lib/libdaxq.so from dax_amd/csrc with hipcc for gfx950.

Cross-compiles without a GPU.  Used by ``__graft_entry__.build()``; the tests, the
smoke run and the benchmark load the library that is already there.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libdaxq.so")
MFMA_RATE = os.path.join(LIBDIR, "mfma_rate")
SOURCES = ["capi.hip", "quant_rows.hip", "fused_rows.hip", "per_tensor.hip", "gemm_w8a8.hip", "gemm_tile256.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-fast-math",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err and verbose:
        print(err, file=sys.stderr)
    return obj


def build(verbose: bool = False) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=len(SOURCES)) as ex:
        objs = list(ex.map(lambda s: _compile(s, verbose), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    # stand-alone microbenchmark behind bench.py's sustained-MFMA-rate figure
    cmd = [HIPCC, *FLAGS, os.path.join(CSRC, "microbench", "mfma_rate.hip"), "-o", MFMA_RATE]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on mfma_rate.hip:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
