"""W8A8 linear throughput at the Wan2.1-14B 720p shapes on one MI355X (INT8 and FP8, one block and 40 layers).

One step = one pass of the quantised-linear hot path over the four linears of a DiT block at M = 75600 tokens
(QKV 5120->15360, out-proj 5120->5120, FFN 5120->13824, FFN 13824->5120): per linear, the per-token activation
quantiser and the MFMA GEMM with the fused epilogue.  Inputs (bf16 activations, pre-quantised weights, scales, bias)
are resident in HBM before the timed region.  Prints ONE JSON line:

  * top level      the INT8 step (the headline configuration)
  * "fp8"          the same step with e4m3fn activations and weights
  * "model40"      INT8, 40 layers x {QKV, out, cross-q at M tokens; cross-k, cross-v at 512 text tokens; FFN up,
                   FFN down} with distinct weights per layer, timed end to end; "attn2_to_out" (the cross-attention
                   output projection of the real block, not part of that list) is timed and reported beside it
  * "wan1_3b"      INT8, the four linears of a Wan2.1-1.3B block at 480p (M = 32760, hidden 1536, FFN 8960)
  * "m9450"        INT8, the 14B step on one GPU's share of the rows under the reference's eight-way sequence
                   parallelism (M = 9450)
  * "config0"      INT8, the single linear the reference's CPU path is quoted on (M = 4096, K = N = 1536): one call of the
                   quantiser + GEMM op per step, eagerly and replayed from a captured HIP graph

each with its own ``roofline`` (GEMM launches, HIP events on the launch stream) and ``cpu_baseline`` (the CPU oracle
on a bounded sample of the same tensors).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only int8|fp8|fp8_e5m2|model40] [--model 14b|1.3b|config0]

Synthetic inputs follow one seeded CPU recipe (seed = index of the linear): X = randn(M, K), 1 % of the columns x 20,
bf16; W = bf16(0.02 randn(N, K)); bias = bf16(0.01 randn(N)); they are copied to the device, and the CPU leg reads the
same tensors.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

M_TOKENS = 75600
TEXT_TOKENS = 512
SHAPES = [("qkv", 5120, 15360), ("out", 5120, 5120), ("ffn_up", 5120, 13824), ("ffn_down", 13824, 5120)]
# The other linear set the reference is quoted on (Wan2.1-1.3B at 480p, 21*30*52 tokens): --model 1.3b.  Not the
# headline workload; its K = N = 1536 linear sits below the MFMA/HBM ridge, so HBM GB/s is reported beside T-op/s.
MODELS = {"14b": ("Wan2.1-14B 720p", "wan2.1_14b_720p", M_TOKENS, SHAPES),
          "1.3b": ("Wan2.1-1.3B 480p", "wan2.1_1.3b_480p", 32760,
                   [("qkv", 1536, 4608), ("out", 1536, 1536), ("ffn_up", 1536, 8960), ("ffn_down", 8960, 1536)]),
          # the single linear the reference's CPU path is quoted on
          "config0": ("single linear 4096 x 1536 -> 1536", "single_4096x1536x1536", 4096, [("linear", 1536, 1536)])}
PEAK_TOPS = 5000.0  # MI355X dense 8-bit MFMA peak, INT8 and FP8
DTYPE_NAME = {"int8": "int8", "fp8": "fp8_e4m3fn", "fp8_e5m2": "fp8_e5m2_x_e4m3fn"}
# L2-miss bytes per GEMM launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE passes over this command
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemm_tile256__wan14b_720p_hbm_traffic.json")


def synth_inputs(m: int, k: int, n: int, seed: int):
    """Seeded synthetic X [m,k], W [n,k], bias [n], all bf16 on the CPU; 1 % of X's columns are outlier channels
    (x 20).  The multiplication by a column vector of 1 / 20 gives the same values as scaling the columns in place."""
    import torch

    g = torch.Generator("cpu").manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    idx = torch.randperm(k, generator=g)[: max(1, round(0.01 * k))]
    col = torch.ones(k)
    col[idx] = 20.0
    x *= col
    x = x.bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    b = (torch.randn(n, generator=g) * 0.01).bfloat16()
    return x, w, b


def gemm_traffic(kind: str):
    """HBM-side bytes per GEMM launch (average of the four 14B shapes) as the committed counter summary holds them."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)[kind]
        return int(rec["bytes_per_launch"])
    except (OSError, KeyError, ValueError):
        return None


def cpu_baseline(kind: str, rows: int, cpu_layers, note: str):
    """The reference's CPU path (oracle: eager quantiser + torch._int_mm / fp32-emulated fp8 matmul + epilogue) on the
    first `rows` tokens of the SAME tensors the GPU step reads.  cpu_layers: [(name, x, w, b)] bf16 CPU tensors."""
    import torch

    from oracle import daxq_oracle as O

    ops_done, t_total = 0.0, 0.0
    for name, x, w, b in cpu_layers:
        xs = x[: min(rows, x.shape[0])]
        if kind == "int8":
            qw, sw = O.weight_quant_int8(w)
            t0 = time.perf_counter()
            O.linear_int8(xs, qw, sw, b, keep_acc=False)
        else:
            qw, sw = O.weight_quant_e4m3(w)
            t0 = time.perf_counter()
            O.linear_e4m3(xs, qw, sw, b, **({"act_dtype": torch.float8_e5m2} if kind == "fp8_e5m2" else {}))
        t_total += time.perf_counter() - t0
        ops_done += 2.0 * xs.shape[0] * w.shape[0] * w.shape[1]
    return {"value": round(ops_done / t_total / 1e12, 3), "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{note}, {t_total:.1f} s, os.cpu_count()={os.cpu_count()}"}


def mfma_sustained():
    """Runs the register-only MFMA microbenchmark (bench/mfma_rate) as a child process: the MFMA rate this board
    sustains under its power limit for constant / uniform-random / workload-like operands."""
    import subprocess

    exe = os.path.join(ROOT, "bench", "mfma_rate")
    if not os.path.exists(exe):
        return None
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    if r.returncode != 0:
        return {"error": r.stderr.strip()[-200:]}
    rows = [json.loads(line) for line in r.stdout.splitlines() if line.startswith("{")]
    out = {}
    for row in rows:
        out.setdefault(row["dtype"], {})[row["data"]] = row["sustained_tops"]
    return out


class Runner:
    """Holds the device-resident operands of a list of linears and times steps over them."""

    def __init__(self, ops, kind):
        self.ops, self.kind = ops, kind
        fp8, e5m2 = kind != "int8", kind == "fp8_e5m2"
        self.fp8 = fp8
        self.act_quant = ops.act_quant_e5m2 if e5m2 else ops.act_quant_e4m3 if fp8 else ops.act_quant_i8
        self.linear = ops.linear_e5m2_e4m3 if e5m2 else ops.linear_e4m3 if fp8 else ops.linear_i8
        self.layers = []  # (name, k, n, x, qw, sw, b)

    def quantise_weight(self, w):
        lo, hi = self.ops.row_minmax(w)
        sw = self.ops.scale_from_minmax(lo, hi, 448.0 if self.fp8 else 127.0)
        qw = (self.ops.quantize_rows_e4m3 if self.fp8 else self.ops.quantize_rows_i8)(w, sw, True)
        return qw, sw

    def add(self, name, x, w_dev, b_dev):
        qw, sw = self.quantise_weight(w_dev)
        self.layers.append((name, w_dev.shape[1], w_dev.shape[0], x, qw, sw, b_dev))

    def add_quantised(self, name, x, qw, sw, b_dev):
        self.layers.append((name, qw.shape[1], qw.shape[0], x, qw, sw, b_dev))

    def step(self, ev=None):
        out = None
        for li, (name, k, n, x, qw, sw, b) in enumerate(self.layers):
            if ev is not None:
                ev[li][0].record()
            xq, sx = self.act_quant(x)
            if ev is not None:
                ev[li][1].record()
            out = self.linear(xq, sx, qw, sw, b)
            if ev is not None:
                ev[li][2].record()
        return out

    def fused_step(self):
        """One op call per linear (quantiser + GEMM behind one dispatch): what the swapped module's forward runs."""
        fused = (self.ops.dynamic_linear_e5m2_e4m3 if self.kind == "fp8_e5m2" else
                 self.ops.dynamic_linear_e4m3 if self.fp8 else self.ops.dynamic_linear_i8)
        out = None
        for (name, k, n, x, qw, sw, b) in self.layers:
            out = fused(x, qw, sw, b)
        return out

    def run_host_bound(self, steps, warmup):
        """For steps of a few tens of microseconds, where event records between the launches would be what is timed: the
        timed region runs `steps` fused steps with nothing in between (-> ms_per_step, value); the kernel durations behind
        `roofline` come from a second pass of the same number of steps with events (run()); a third figure replays the
        step from a captured HIP graph (what a serving loop that cannot afford the host's launch time does)."""
        import torch

        for _ in range(warmup):
            self.fused_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            self.fused_step()
        torch.cuda.synchronize()
        ms_eager = (time.perf_counter() - t0) * 1e3 / steps
        res = self.run(steps, 2)
        res["ms_per_step_with_events"] = res["ms_per_step"]
        res["ms_per_step"] = ms_eager
        res["value"] = res["total_ops"] / (ms_eager * 1e-3) / 1e12
        res["warmup"] = warmup
        # graph replay: capture one step on a side stream, replay `steps` times
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self.fused_step()
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                self.fused_step()
            for _ in range(3):
                graph.replay()
            side.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                graph.replay()
            side.synchronize()
            res["ms_per_step_graph_replay"] = (time.perf_counter() - t0) * 1e3 / steps
            # the GEMM kernel's own duration: 20 launches on pre-quantised rows captured into one graph, so that no host
            # time sits between them (events around single launches from Python would time the host's launch gaps)
            per = {}
            for (name, k, n, x, qw, sw, b) in self.layers:
                xq, sx = self.act_quant(x)
                self.linear(xq, sx, qw, sw, b)
                side.synchronize()
                g2 = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g2, stream=side):
                    for _ in range(20):
                        self.linear(xq, sx, qw, sw, b)
                g2.replay()
                side.synchronize()
                a, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(side)
                for _ in range(5):
                    g2.replay()
                e.record(side)
                side.synchronize()
                per[name] = a.elapsed_time(e) / 100.0
            gemm_ms = sum(per.values())
            res["gemm_ms"] = gemm_ms
            res["achieved"] = res["total_ops"] / (gemm_ms * 1e-3) / 1e12
            for name, ms in per.items():
                e_ = res["per_linear"][name]
                e_["gemm_ms"] = round(ms, 5)
                e_["gemm_tops"] = round(2.0 * e_["rows"] * e_["n"] * e_["k"] / (ms * 1e-3) / 1e12, 1)
                e_["gemm_gbps"] = round((e_["rows"] * e_["k"] + 4.0 * e_["rows"] + e_["n"] * e_["k"] + 6.0 * e_["n"] + 2.0 * e_["rows"] * e_["n"]) / (ms * 1e-3) / 1e9, 1)
                e_["gemm_hbm_frac"] = round(e_["gemm_gbps"] / 8000.0, 4)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        return res

    def run(self, steps, warmup):
        import torch

        for _ in range(warmup):
            self.step()
        torch.cuda.synchronize()
        evs = [[[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in self.layers] for _ in range(steps)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for s in range(steps):
            self.step(evs[s])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms_per_step = (t1 - t0) * 1e3 / steps
        total_ops = sum(2.0 * x.shape[0] * n * k for _, k, n, x, *_r in self.layers)
        per, gemm_ms, quant_ms = {}, 0.0, 0.0
        for li, (name, k, n, x, *_rest) in enumerate(self.layers):
            q_ms = sum(evs[s][li][0].elapsed_time(evs[s][li][1]) for s in range(steps)) / steps
            g_ms = sum(evs[s][li][1].elapsed_time(evs[s][li][2]) for s in range(steps)) / steps
            e = per.setdefault(name, {"k": k, "n": n, "rows": x.shape[0], "launches": 0, "quant_ms": 0.0, "gemm_ms": 0.0})
            e["launches"] += 1
            e["quant_ms"] += q_ms
            e["gemm_ms"] += g_ms
            gemm_ms += g_ms
            quant_ms += q_ms
        for e in per.values():
            rows, k, n, cnt = e["rows"], e["k"], e["n"], e["launches"]
            e["gemm_tops"] = round(cnt * 2.0 * rows * n * k / (e["gemm_ms"] * 1e-3) / 1e12, 1)
            e["quant_gbps"] = round(cnt * (3.0 * rows * k + 4.0 * rows) / (e["quant_ms"] * 1e-3) / 1e9, 1)
            # algorithmic bytes of the GEMM launch: both operands, scales, bias, the bf16 output
            e["gemm_gbps"] = round(cnt * (rows * k + 4.0 * rows + n * k + 6.0 * n + 2.0 * rows * n) / (e["gemm_ms"] * 1e-3) / 1e9, 1)
            e["gemm_hbm_frac"] = round(e["gemm_gbps"] / 8000.0, 4)  # algorithmic bytes of the launch against 8 TB/s
            e["quant_ms"], e["gemm_ms"] = round(e["quant_ms"], 4), round(e["gemm_ms"], 4)
        achieved = total_ops / (gemm_ms * 1e-3) / 1e12
        return {"ms_per_step": ms_per_step, "total_ops": total_ops, "value": total_ops / (ms_per_step * 1e-3) / 1e12,
                "achieved": achieved, "gemm_ms": gemm_ms, "quant_ms": quant_ms, "per_linear": per, "steps": steps, "warmup": warmup}


def roofline(res, kind, kernel, traffic):
    return {"bound": "mfma", "achieved": round(res["achieved"], 2), "peak": PEAK_TOPS,
            "unit": "TOP/s" if kind == "int8" else "TFLOP/s", "frac": round(res["achieved"] / PEAK_TOPS, 4), "traffic": traffic,
            "kernel": kernel, "gemm_ms_per_step": round(res["gemm_ms"], 4), "quant_ms_per_step": round(res["quant_ms"], 4)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--only", choices=["int8", "fp8", "fp8_e5m2", "model40"], default=None,
                    help="run one part only (profiling); default: the INT8 step as the headline with the FP8 step and "
                         "the 40-layer INT8 workload as sub-records.  fp8_e5m2: e5m2 activations against e4m3fn weights, "
                         "the default pairing of the reference's FP8 qconfig factory")
    ap.add_argument("--model", choices=sorted(MODELS), default="14b",
                    help="which linear set: 14b (the headline workload), 1.3b (M = 32760, hidden 1536, FFN 8960) or "
                         "config0 (one linear, M = 4096, K = N = 1536); the sub-records exist for 14b only")
    ap.add_argument("--variant", type=int, default=0, help="GEMM kernel selection for comparisons (0 = library default)")
    ap.add_argument("--tile-group", type=int, default=0, help="tile-order group depth (0 = library default)")
    ap.add_argument("--tile-order", type=int, default=0, help="tile order of the 256x256 kernels: 0 = library default, 1 = row groups, 2 = banded patches")
    ap.add_argument("--m", type=int, default=0, help="tokens (0 = the model's own count)")
    ap.add_argument("--linear", default=None,
                    help="comma-separated names of the model's linears to keep (qkv, out, ffn_up, ffn_down): a step of one "
                         "linear repeats the same weight, i.e. measures it warm")
    ap.add_argument("--cpu-rows", type=int, default=0, help="tokens in the CPU-baseline sample (0 = pick for 10-30 s)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-mfma-ceiling", action="store_true")
    ap.add_argument("--no-producers", action="store_true")
    ap.add_argument("--kv-fused", action="store_true", help="40-layer workload: the text tokens' k and v projections as one N-concatenated launch")
    ap.add_argument("--no-sub-records", action="store_true", help="leave out the wan1_3b / m9450 / config0 sub-records of the default run")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (reference point for HBM traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus must be 1 (the path shards by token rows, "
                 "no multi-GPU figure is produced)")

    import torch

    import dax_amd.ops as ops
    from dax_amd import _capi

    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    _capi.require_gfx950(0)
    if args.variant or args.tile_group or args.tile_order:
        _capi.debug_select_gemm(args.variant)
        if args.tile_group:
            _capi.debug_select_gemm(1000 + args.tile_group)
        if args.tile_order:
            _capi.debug_select_gemm(2000 + args.tile_order)
    dev = torch.device("cuda:0")
    model_name, model_tag, m_model, shapes = MODELS[args.model]
    m = args.m or m_model
    if args.linear:
        keep = args.linear.split(",")
        unknown = [nm for nm in keep if nm not in [s_[0] for s_ in shapes]]
        if unknown:
            sys.exit(f"bench.py: --linear {unknown}: the {args.model} set has {[s_[0] for s_ in shapes]}")
        shapes = [s_ for s_ in shapes if s_[0] in keep]
    full = args.model == "14b" and m == M_TOKENS and not args.linear
    parts = [args.only] if args.only else (["int8", "fp8", "model40"] if full else ["int8"])
    if "model40" in parts and not full:
        sys.exit("bench.py: the 40-layer workload is defined for --model 14b at its own token count")
    head_kind = parts[0] if parts[0] != "model40" else "int8"

    # ---- synthetic inputs: one seeded CPU recipe per linear, copied to HBM; the CPU leg reads the same tensors
    t_gen = time.perf_counter()
    cpu_layers, dev_layers = [], []
    for i, (name, k, n) in enumerate(shapes):
        x, w, b = synth_inputs(m, k, n, seed=i)
        cpu_layers.append((name, x, w, b))
        dev_layers.append((name, x.to(dev), w.to(dev), b.to(dev)))
    t_gen = time.perf_counter() - t_gen

    info = _capi.device_info(0)
    shape_txt = ", ".join(f"{nm} {k}->{n}" for nm, k, n in shapes)
    per_lin_txt = "per linear: per-token act quant + MFMA GEMM + fused scale/bias/bf16 epilogue"
    def block_record(kind, name_, tag_, m_, shapes_, dev_layers_, cpu_layers_, steps_, warmup_, traffic, cpu_rows, host_bound=False):
        """One step over the linears of `shapes_` at m_ tokens: runs it, and returns the record with roofline and cpu_baseline."""
        r = Runner(ops, kind)
        for name, x, w, b in dev_layers_:
            r.add(name, x, w, b)
        res = r.run_host_bound(steps_, warmup_) if host_bound else r.run(steps_, warmup_)
        del r
        txt = ", ".join(f"{nm} {k}->{n}" for nm, k, n in shapes_)
        rec = {
            "metric": f"w8a8_linear_tops_{tag_}_{kind}",
            "value": round(res["value"], 2), "unit": "TOPS", "ms_per_step": round(res["ms_per_step"], 4),
            "steps": res["steps"], "warmup": res["warmup"], "dtype": DTYPE_NAME[kind],
            "config": {"workload": f"{name_} linear set, {kind.upper()} W8A8, M={m_} tokens: {txt}; {per_lin_txt}",
                       "gemm_variant": args.variant},
            "pct_of_mfma_peak": round(100.0 * res["value"] / PEAK_TOPS, 2),
            "roofline": roofline(res, kind, ("gemm_tile256s5_kernel" if kind == "int8" else "gemm_tile_fp8_kernel") +
                                 f", average launch over the {len(shapes_)} shape(s); 8-bit ops counted as 2*M*N*K", traffic),
            "per_linear": res["per_linear"],
        }
        if host_bound:
            rec["ms_per_step_graph_replay"] = round(res["ms_per_step_graph_replay"], 4)
            rec["value_graph_replay"] = round(res["total_ops"] / (res["ms_per_step_graph_replay"] * 1e-3) / 1e12, 2)
            rec["config"]["step"] = ("one call of the quantiser + GEMM op per linear with nothing in between (the step is the host's "
                                     "launch time); roofline = the GEMM kernel's own duration, 20 launches captured into one HIP graph "
                                     "and replayed between two events; graph replay = the whole step captured once into a HIP graph")
        if not args.no_cpu_baseline:
            rows = min(cpu_rows, m_)
            rec["cpu_baseline"] = cpu_baseline(kind, rows, cpu_layers_,
                                               f"first {rows} of {m_} tokens of each of the {len(shapes_)} linears (same tensors as the GPU step)")
        return rec

    blocks = {}
    for kind in [p for p in parts if p != "model40"]:
        blocks[kind] = block_record(kind, model_name, model_tag, m, shapes, dev_layers, cpu_layers, args.steps, args.warmup,
                                    gemm_traffic(kind) if full else None, args.cpu_rows or (49152 if kind == "int8" else 24576),
                                    host_bound=args.model == "config0")

    model40 = None
    if "model40" in parts:
        # Weights of one layer from the seeded CPU recipe (seeds 0-3 above, 4-7 for cross-q / k / v and the
        # cross-attention output projection); layer l uses them rolled by l output channels (rows of W, scales and
        # bias together): 40 distinct weight sets in HBM of the same distribution.
        text, _, _ = synth_inputs(TEXT_TOKENS, 5120, 8, seed=100)
        text_dev = text.to(dev)
        x5120, x13824 = dev_layers[0][1], dev_layers[3][1]
        base = {name: (w, b) for name, _x, w, b in dev_layers}
        cpu_extra = {}
        for j, name in enumerate(("cross_q", "cross_k", "cross_v", "attn2_to_out")):
            _x, w, b = synth_inputs(8, 5120, 5120, seed=4 + j)
            cpu_extra[name] = (w, b)
            base[name] = (w.to(dev), b.to(dev))
        order = [("qkv", x5120), ("out", x5120), ("cross_q", x5120), ("cross_k", text_dev), ("cross_v", text_dev),
                 ("ffn_up", x5120), ("ffn_down", x13824)]
        if args.kv_fused:
            # k and v of the text tokens as ONE launch against the N-concatenated weight (per-channel weight scales and
            # per-token activation scales make it bit-identical to the two launches; the self-attention QKV of this
            # list is the same construction)
            base["cross_kv"] = (torch.cat([base["cross_k"][0], base["cross_v"][0]], 0), torch.cat([base["cross_k"][1], base["cross_v"][1]], 0))
            order = [o for o in order if o[0] not in ("cross_k", "cross_v")]
            order.insert(3, ("cross_kv", text_dev))
        r = Runner(ops, "int8")
        q0 = {name: r.quantise_weight(base[name][0]) for name, _ in order}
        for layer in range(40):
            for name, x in order:
                qw, sw = q0[name]
                r.add_quantised(name, x, torch.roll(qw, layer, 0), torch.roll(sw, layer, 0), torch.roll(base[name][1], layer, 0))
        steps40 = max(2, args.steps // 5)
        res = r.run(steps40, 1)
        del r
        model40 = {
            "metric": f"w8a8_linear_tops_{model_tag}_int8_40_layers",
            "value": round(res["value"], 2), "unit": "TOPS", "ms_per_step": round(res["ms_per_step"], 3),
            "steps": steps40, "warmup": 1, "dtype": "int8", "total_pops": round(res["total_ops"] / 1e15, 4),
            "config": {"workload": f"Wan2.1-14B 720p, 40 layers x (QKV 5120->15360, out, cross-q 5120->5120 at M={m}; cross-k, "
                                   f"cross-v 5120->5120 at {TEXT_TOKENS} text tokens; FFN 5120->13824, 13824->5120), INT8 W8A8, every "
                                   "linear with its own per-token act quant; one seeded weight set, rolled by the layer index "
                                   "along the output channels to give 40 distinct sets"},
            "pct_of_mfma_peak": round(100.0 * res["value"] / PEAK_TOPS, 2),
            "roofline": roofline(res, "int8", "all GEMM launches of the step (the 512-token ones run the 128x128-tile form)", None),
            "per_linear": res["per_linear"],
        }
        # the real block's cross-attention output projection (5120 -> 5120 at M tokens), not in the list above
        r = Runner(ops, "int8")
        r.add("attn2_to_out", x5120, *base["attn2_to_out"])
        ra = r.run(max(4, args.steps), 2)
        del r
        model40["attn2_to_out"] = {
            "ms_per_call": round(ra["ms_per_step"], 4), "gemm_ms": round(ra["gemm_ms"], 4), "quant_ms": round(ra["quant_ms"], 4),
            "gemm_tops": round(ra["achieved"], 1), "tops": round(ra["value"], 1),
            "note": "x40 it adds %.1f ms and %.3f P-op to the 40-layer step (then %.1f TOPS)" % (
                40 * ra["ms_per_step"], 40 * ra["total_ops"] / 1e15,
                (res["total_ops"] + 40 * ra["total_ops"]) / ((res["ms_per_step"] + 40 * ra["ms_per_step"]) * 1e-3) / 1e12)}
        if not args.no_cpu_baseline:
            rows = min(args.cpu_rows or 24576, m)
            one = [(n_, x_, w_, b_) for n_, x_, w_, b_ in cpu_layers if n_ in ("qkv", "out")]
            one.append(("cross_q", cpu_layers[0][1], *cpu_extra["cross_q"]))
            one += [("cross_k", text, *cpu_extra["cross_k"]), ("cross_v", text, *cpu_extra["cross_v"])]
            one += [(n_, x_, w_, b_) for n_, x_, w_, b_ in cpu_layers if n_ in ("ffn_up", "ffn_down")]
            model40["cpu_baseline"] = cpu_baseline(
                "int8", rows, one, f"ONE layer of the 40 (7 linears; first {rows} of {m} tokens, all {TEXT_TOKENS} text tokens); "
                                   "the 40 layers cost the same each, so the rate stands for the whole step")

    # ---- the other configurations the reference is quoted on, as sub-records of the default run (INT8)
    extra = {}
    if full and not args.only and not args.no_sub_records:
        # one GPU's share of the rows under the reference's eight-way sequence parallelism: the first 9450 tokens
        sl_dev = [(nm, x[:9450], w, b) for nm, x, w, b in dev_layers]
        sl_cpu = [(nm, x[:9450], w, b) for nm, x, w, b in cpu_layers]
        # (steps of 1 - 2 ms: at least 40 warm-up and 40 timed ones, so that the card is back at its clocks after the
        # host-side work in front of the record and the timed region is long against a launch)
        sub_steps, sub_warmup = max(args.steps, 40), max(args.warmup, 40)
        extra["m9450"] = block_record("int8", model_name + ", 1/8 of the rows", model_tag + "_m9450", 9450, shapes, sl_dev, sl_cpu,
                                      sub_steps, sub_warmup, None, 4096)
        for key in ("1.3b", "config0"):
            name_, tag_, m_, shapes_ = MODELS[key]
            cl, dl = [], []
            for i, (nm, k, n) in enumerate(shapes_):
                x, w, b = synth_inputs(m_, k, n, seed=i)
                cl.append((nm, x, w, b))
                dl.append((nm, x.to(dev), w.to(dev), b.to(dev)))
            small = key == "config0"
            extra["config0" if small else "wan1_3b"] = block_record(
                "int8", name_, tag_, m_, shapes_, dl, cl, 200 if small else sub_steps, 20 if small else sub_warmup, None,
                4096 if small else 16384, host_bound=small)
            del cl, dl

    if args.calib_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    if head_kind in blocks:
        head = blocks.pop(head_kind)
    else:  # --only model40
        head = dict(model40)
        model40 = None
    res = {
        "metric": head["metric"], "value": head["value"], "unit": "TOPS", "n_gpus": 1, "steps": head["steps"],
        "warmup": head["warmup"], "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic", "config": head["config"],
        "pct_of_mfma_peak": head["pct_of_mfma_peak"], "roofline": head["roofline"],
    }
    if "cpu_baseline" in head:
        res["cpu_baseline"] = head["cpu_baseline"]
    for key in ("per_linear", "attn2_to_out", "total_pops", "ms_per_step_graph_replay", "value_graph_replay"):
        if key in head:
            res[key] = head[key]
    for kind, rec in blocks.items():
        res["fp8" if kind == "fp8" else kind] = rec
    if model40 is not None:
        res["model40"] = model40
    res.update(extra)
    res["device"] = {"arch": info["arch"], "cu_count": info["cu_count"], "max_clock_mhz": info["clock_khz"] / 1000.0}
    res["input_generation_s"] = round(t_gen, 1)

    # ---- the fused producer + quantiser kernels (outside the timed step): LayerNorm multiply-add in front of
    #      the K=5120 linears, GELU-tanh in front of the 13824 -> 5120 one; algorithmic bytes 3 per element
    def timed(fn, reps=20):
        # The first calls pay for fresh allocations, and after the host-side work above the card has dropped its clocks:
        # 0.29 ms for the LayerNorm form after two idle seconds against 0.235 ms in a busy stream.  Warm for 50 ms.
        fn()
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        while time.perf_counter() - t_warm < 0.05:
            for _ in range(10):
                fn()
            torch.cuda.synchronize()
        a, b2 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b2.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b2) / reps

    if not args.no_producers:
        hidden, ffn = shapes[0][1], shapes[-1][1]
        xs = {k: x for _n, x, _w, _b in dev_layers for k in [x.shape[1]]}
        mul = 1 + 0.1 * torch.randn(1, hidden, device=dev)
        add = 0.1 * torch.randn(1, hidden, device=dev)
        prod = {}
        kinds = [k_ for k_ in dict.fromkeys([head_kind] + list(blocks)) if k_ in ("int8", "fp8", "fp8_e5m2")] or ["int8"]
        for kind in kinds:
            fmt = {"int8": "i8", "fp8": "e4m3", "fp8_e5m2": "e5m2"}[kind]
            ln_ms = timed(lambda: getattr(ops, "layernorm_act_quant_" + fmt)(xs[hidden], mul, add, m, 1e-6))
            ge_ms = timed(lambda: getattr(ops, "gelu_tanh_act_quant_" + fmt)(xs[ffn]))
            prod[kind] = {
                f"layernorm_modulate_quant_k{hidden}": {"ms": round(ln_ms, 4), "gbps": round(3.0 * m * hidden / (ln_ms * 1e-3) / 1e9, 1)},
                f"gelu_tanh_quant_k{ffn}": {"ms": round(ge_ms, 4), "gbps": round(3.0 * m * ffn / (ge_ms * 1e-3) / 1e9, 1)}}
        prod["hbm_peak_gbps"] = 8000.0
        res["fused_producers"] = prod
    if not args.no_mfma_ceiling:
        sus = mfma_sustained()
        if sus and "error" not in sus:
            res["mfma_sustained"] = {
                "unit": "TOPS", **sus,
                "note": "register-only MFMA loop, no memory traffic: the rate the board holds under its power limit "
                        "depends on operand bit activity; 'workload' uses this benchmark's value distribution"}
            want = "int8" if head["dtype"] == "int8" else "fp8_e4m3fn"
            if want in sus and "workload" in sus[want]:
                res["roofline"]["gemm_frac_of_workload_ceiling"] = round(head["roofline"]["achieved"] / sus[want]["workload"], 4)
            if "fp8" in res and "fp8_e4m3fn" in sus and "workload" in sus["fp8_e4m3fn"]:
                res["fp8"]["roofline"]["gemm_frac_of_workload_ceiling"] = round(
                    res["fp8"]["roofline"]["achieved"] / sus["fp8_e4m3fn"]["workload"], 4)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
