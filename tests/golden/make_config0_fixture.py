"""Writes tests/golden/config0_int8.json: digests and a corner of every tensor of benchmark config 0
(INT8, M=4096, K=N=1536, seed 0) as the CPU oracle computes them.

The reference ships no golden vectors for this path, so this fixture is generated from the oracle
(oracle/daxq_oracle.py), not from the reference.  It freezes the oracle's results: a later torch
version or an edit of the oracle that changes a single bit of the quantised activations, the
accumulators or the bf16 outputs fails tests/test_golden.py, and the GPU test compares the HIP path
with the same digests without running the oracle.  Run from the repository root:
    python tests/golden/make_config0_fixture.py
"""
import hashlib
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
from oracle import daxq_oracle as O  # noqa: E402

M, K, N, SEED = 4096, 1536, 1536, 0


def digest(t: torch.Tensor) -> str:
    raw = t.detach().contiguous().cpu()
    raw = raw.view(torch.uint8) if raw.dtype in (torch.float8_e4m3fn, torch.int8) else raw
    return hashlib.sha256(raw.numpy().tobytes() if raw.dtype != torch.bfloat16 else raw.view(torch.int16).numpy().tobytes()).hexdigest()


def corner(t: torch.Tensor, r=4, c=8):
    t = t.detach().cpu()
    if t.dim() == 1:
        return t[:c].float().tolist()
    return t[:r, :c].float().tolist()


def compute():
    x, w, b = O.make_inputs(M, K, N, seed=SEED)
    qw, sw = O.weight_quant_int8(w)
    r = O.linear_int8(x, qw, sw, b, keep_acc=True)
    tensors = {"x": x, "w": w, "bias": b, "qweight": qw, "weight_scale": sw.reshape(-1), "xq": r["xq"],
               "sx": r["sx"].reshape(-1), "acc": r["acc"], "out": r["out"]}
    fx, fsw = O.act_quant_e4m3(x), O.weight_quant_e4m3(w)
    tensors.update({"xq_e4m3": fx[0], "sx_e4m3": fx[1].reshape(-1), "qweight_e4m3": fsw[0], "weight_scale_e4m3": fsw[1].reshape(-1)})
    return tensors


def main():
    t = compute()
    out = {"config": {"m": M, "k": K, "n": N, "seed": SEED, "torch": torch.__version__},
           "sha256": {k: digest(v) for k, v in t.items()},
           "corner": {k: corner(v) for k, v in t.items()}}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config0_int8.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
