"""Vendor-library 8-bit GEMMs on the benchmark's shapes and data, as a yardstick beside bench.py's figures.

Not part of the product: times torch._int_mm (int32 output, no epilogue) and torch._scaled_mm (row-wise and per-tensor
scales, bf16 output) on the same quantised operands the daxq GEMM reads, and the daxq GEMM itself in the same
process, alternating, so that all numbers come from one box in one power state.  Prints one JSON line.

    python3 bench/vendor_yardstick.py [--reps 10]
"""
import argparse
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--reps", type=int, default=10)
    args = ap.parse_args()
    import torch

    import bench
    import dax_amd.ops as ops

    dev = torch.device("cuda:0")
    m = bench.M_TOKENS

    def timeit(f):
        for _ in range(3):
            f()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(args.reps):
            f()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / args.reps

    out = {"unit": "T-op/s (2*M*N*K per call)", "m": m, "reps": args.reps, "torch": torch.__version__, "shapes": {}}
    for i, (name, k, n) in enumerate(bench.SHAPES):
        x, w, b = bench.synth_inputs(m, k, n, seed=i)
        x, w, b = x.to(dev), w.to(dev), b.to(dev)
        ops_ = 2.0 * m * n * k
        rec = {}
        # INT8 operands from the product's quantisers
        xq, sx = ops.act_quant_i8(x)
        lo, hi = ops.row_minmax(w)
        sw = ops.scale_from_minmax(lo, hi, 127.0)
        wq = ops.quantize_rows_i8(w, sw, True)
        cands = {"daxq_linear_i8 (scales, bias, bf16 out)": lambda: ops.linear_i8(xq, sx, wq, sw, b)}
        try:
            wt = wq.t()
            torch._int_mm(xq, wt)
            cands["torch._int_mm (int32 out, no epilogue)"] = lambda: torch._int_mm(xq, wt)
        except Exception as ex:  # noqa: BLE001
            rec["torch._int_mm"] = "failed: " + repr(ex)[:160]
        # FP8 operands
        xf, sxf = ops.act_quant_e4m3(x)
        sw8 = ops.scale_from_minmax(lo, hi, 448.0)
        wf = ops.quantize_rows_e4m3(w, sw8, True)
        cands["daxq_linear_e4m3 (scales, bias, bf16 out)"] = lambda: ops.linear_e4m3(xf, sxf, wf, sw8, b)
        xf8, wf8t = xf.view(torch.float8_e4m3fn), wf.view(torch.float8_e4m3fn).t()
        sa, sb = sxf.view(-1, 1).contiguous(), sw8.view(1, -1).contiguous()
        one = torch.ones((), device=dev)
        for label, kw in (("torch._scaled_mm row-wise scales + bias", dict(scale_a=sa, scale_b=sb, bias=b)),
                          ("torch._scaled_mm per-tensor scales + bias", dict(scale_a=one, scale_b=one, bias=b))):
            try:
                torch._scaled_mm(xf8, wf8t, out_dtype=torch.bfloat16, use_fast_accum=True, **kw)
                cands[label] = (lambda kw=kw: torch._scaled_mm(xf8, wf8t, out_dtype=torch.bfloat16, use_fast_accum=True, **kw))
            except Exception as ex:  # noqa: BLE001
                rec[label] = "failed: " + repr(ex)[:160]
        best = {c: float("inf") for c in cands}
        for _ in range(2):  # alternate, keep the better of two rounds
            for c, f in cands.items():
                best[c] = min(best[c], timeit(f))
        for c, t in best.items():
            rec[c] = {"ms": round(t, 4), "tops": round(ops_ / t / 1e9, 1)}
        out["shapes"][f"{name} {k}->{n}"] = rec
        del x, w, xq, wq, xf, wf
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
