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
ROOT = os.path.dirname(HERE)
MFMA_RATE = os.path.join(ROOT, "bench", "mfma_rate")
SOURCES = ["capi.hip", "quant_rows.hip", "quant_blocks.hip", "fused_rows.hip", "per_tensor.hip", "gemm_w8a8.hip", "gemm_tile256.hip", "gemm_tile_fp8.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-fast-math",
    # packed-FP32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


# Every source but the fused producers is compiled without floating-point contraction: a multiply followed by an
# add (INT8 / FP8 epilogues: scale, scale, bias) or by a narrowing convert (fp16 outputs) must round once per
# operation, as the reference's op sequence does; contraction turns them into an fma or a mixed-precision fma with a
# single rounding.  fused_rows.hip (LayerNorm / GELU statistics, compared at a stated tolerance) keeps its fmas.
NO_CONTRACT = {"quant_rows.hip", "quant_blocks.hip", "per_tensor.hip", "gemm_w8a8.hip", "gemm_tile256.hip", "gemm_tile_fp8.hip"}


def _compile(src: str, verbose: bool) -> str:
    obj = os.path.join(LIBDIR, os.path.splitext(src)[0] + ".o")
    extra = ["-ffp-contract=off"] if src in NO_CONTRACT else []
    cmd = [HIPCC, *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
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
    cmd = [HIPCC, *FLAGS, os.path.join(ROOT, "bench", "mfma_rate.hip"), "-o", MFMA_RATE]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on mfma_rate.hip:\n{r.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
