"""How the swapped module sits in a caller's runtime: inside a traced graph, on a stream that is not
the default one, and inside a captured HIP graph that is replayed.

The reference module is used under ``torch.compile`` (functional.py:33-36) and runs on whatever stream
is current while a communication stream is busy (attn_adapter.py:102-160).  Each test compares the
result with the same module called eagerly on the default stream, bit for bit (same kernels, same inputs).
"""
import pytest
import torch
from torch import nn

from tests.util import bf16_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _fresh_compiler_cache():
    """Every test here compiles the same Sequential.forward code object for another module; the compiler keeps at
    most eight specialisations per code object and refuses the ninth under fullgraph=True."""
    torch._dynamo.reset()
    yield


def _mlp(k, n, fp8, seed):
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig,
                                                    get_dynamic_int8_per_token_act_per_channel_weight_qconfig)

    torch.manual_seed(seed)
    model = nn.Sequential(nn.Linear(k, n), nn.GELU(approximate="tanh"), nn.Linear(n, k)).bfloat16().to("cuda")
    cfg = (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(activation_dtype=torch.float8_e4m3fn)
           if fp8 else get_dynamic_int8_per_token_act_per_channel_weight_qconfig())
    quantize_dynamic(model, {"": cfg})
    return model


def _input(m, k, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    return torch.randn(2, m, k, generator=g).bfloat16().to("cuda")


def _same(a, b):
    return (bf16_bits(a) == bf16_bits(b)).all()


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("k", [384, 392])  # 392: the weight is zero-padded to 512 columns inside the graph
@pytest.mark.parametrize("fp8", [False, True])
def test_traced_graph_matches_eager(fp8, k, backend):
    """One graph without breaks: every op has a fake kernel, so the tracer sees shapes and dtypes only.  With the
    reference's own setting (torch.compile's default backend, functional.py:33-36) the code generator compiles what
    lies between the linears (the GELU here) and calls the daxq ops as they are."""
    if backend == "inductor":
        pytest.importorskip("triton")
    model = _mlp(k, 520, fp8, seed=1)
    x = _input(300, k, seed=2)
    ref = model(x)
    traced = torch.compile(model, backend=backend, fullgraph=True)
    out = traced(x)
    assert out.shape == ref.shape and out.dtype == torch.bfloat16
    assert _same(out, ref)
    x2 = _input(300, k, seed=3)
    assert _same(traced(x2), model(x2))


@pytest.mark.parametrize("fp8", [False, True])
def test_few_rows_traced_and_in_a_captured_graph(fp8):
    """Ten rows: the op quantises into a 128-row buffer and returns the first ten rows of the tiled kernel's output.
    Traced (the fake kernel promises a [10, N] tensor) and captured into a HIP graph, every call equals eager."""
    model = _mlp(384, 520, fp8, seed=21)
    x = _input(5, 384, seed=22)
    ref = model(x)
    traced = torch.compile(model, backend="aot_eager", fullgraph=True)
    assert _same(traced(x), ref)
    static_x = x.clone()
    model(static_x)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = model(static_x)
    for seed in (23, 24, 25):
        x2 = _input(5, 384, seed=seed)
        want = model(x2)
        torch.cuda.synchronize()
        static_x.copy_(x2)
        graph.replay()
        torch.cuda.synchronize()
        assert _same(static_out, want), f"replay with seed {seed} differs from eager"


@pytest.mark.parametrize("fp8", [False, True])
def test_compiled_with_graph_replay_matches_eager(fp8):
    """torch.compile(mode="reduce-overhead"): the generated code and the daxq ops are captured into a HIP graph by
    the compiler's runtime and replayed from the third call on; every call equals eager."""
    pytest.importorskip("triton")
    model = _mlp(384, 520, fp8, seed=12)
    compiled = torch.compile(model, mode="reduce-overhead", fullgraph=True)
    for seed in (13, 14, 15, 16, 17):
        x = _input(300, 384, seed=seed)
        ref = model(x)
        out = compiled(x).clone()   # the replayed graph owns its output buffer
        torch.cuda.synchronize()
        assert _same(out, ref), f"call with seed {seed} differs from eager"


@pytest.mark.parametrize("fp8", [False, True])
def test_side_stream_runs_beside_a_busy_default_stream(fp8):
    """The kernels go to the stream that is current for the input's device, not to the default one: the
    result is ready while a long spin kernel still holds the default stream."""
    model = _mlp(512, 768, fp8, seed=4)
    x = _input(700, 512, seed=5)
    ref = model(x)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    blocker_done, side_done = torch.cuda.Event(), torch.cuda.Event()
    # a spin kernel of about half a second on the default stream; its counter's rate is measured first
    t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0.record()
    torch.cuda._sleep(1_000_000)
    t1.record()
    t1.synchronize()
    ticks_per_ms = 1_000_000 / max(t0.elapsed_time(t1), 1e-3)
    torch.cuda._sleep(int(min(500 * ticks_per_ms, 4e9)))
    blocker_done.record()
    with torch.cuda.stream(side):
        out = model(x)
        side_done.record()
    side_done.synchronize()
    finished_first = not blocker_done.query()
    torch.cuda.synchronize()
    assert _same(out, ref)
    assert finished_first, "the linear waited for the default stream"


@pytest.mark.parametrize("fp8", [False, True])
def test_captured_graph_replays_match_eager(fp8):
    """Capture the two linears (and a LayerNorm + quantiser launch in front) once, replay with new input
    contents, with eager work and synchronisations between the replays; every replay must equal eager."""
    import dax_amd.ops as ops

    k, n, m = 640, 1024, 520
    model = _mlp(k, n, fp8, seed=6)
    lin0 = model[0]
    ln_quant = ops.layernorm_act_quant_e4m3 if fp8 else ops.layernorm_act_quant_i8
    from dax_amd.quant.nn.dynamic.linear import QuantizedActivation

    def run(x):
        q, s, _ = ln_quant(x.view(-1, k), None, None, x.numel() // k, 1e-6, False)
        y = lin0(QuantizedActivation(q, s, x.shape[:-1], k, lin0.input_dtype))
        return model[2](model[1](y))

    static_x = _input(m, k, seed=7)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # first calls set kernel attributes: keep them outside the capture
        for _ in range(2):
            run(static_x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_out = run(static_x)
    for seed in (8, 9, 10, 11):
        new_x = _input(m, k, seed=seed)
        eager = run(new_x)
        torch.cuda.synchronize()
        static_x.copy_(new_x)
        graph.replay()
        torch.cuda.synchronize()
        assert _same(static_out, eager), f"replay with seed {seed} differs from eager"


def test_split_k_shape_captured_on_a_stream_that_already_has_a_workspace():
    """M = 256, N = K = 5120: eagerly this INT8 launch cuts K into ranges and goes through a workspace that belongs
    to the stream.  A capture on that stream must not record the workspace's address (a graph may replay beside another
    one, or after a larger eager request has replaced the workspace): under capture the plain launch runs, whose INT8
    results are the same bits.  The workspace is then outgrown eagerly, and every replay still equals eager."""
    import dax_amd.ops as ops
    from oracle import daxq_oracle as O

    m, n, k = 256, 5120, 5120
    assert ops._capi.lib().daxq_linear_splitk_choice(m, n, k) > 1
    x, w, b = O.make_inputs(m, k, n, seed=77)
    dev = torch.device("cuda")
    wd, bd = w.to(dev), b.to(dev)
    lo, hi = ops.row_minmax(wd)
    sw = ops.scale_from_minmax(lo, hi, 127.0)
    qw = ops.quantize_rows_i8(wd, sw, True)

    def run(xd):
        return ops.dynamic_linear_i8(xd, qw, sw, bd)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    static_x = x.to(dev)
    with torch.cuda.stream(side):
        eager0 = run(static_x)          # split-K: this stream now owns a workspace
        side.synchronize()
        key = (dev.index if dev.index is not None else torch.cuda.current_device(), side.cuda_stream)
        assert key in ops._splitk_ws
        ws_before = ops._splitk_ws[key]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = run(static_x)
        # an explicit request for more ranges than the first workspace holds replaces it; the old one stays alive
        big_m = 1024
        xb, _, _ = O.make_inputs(big_m, k, n, seed=78)
        xq, sx = ops.act_quant_i8(xb.to(dev))
        need = ops._capi.lib().daxq_linear_splitk_workspace_bytes(big_m, n, 4)
        assert need > ws_before.numel()
        big = ops.linear_w8a8_splitk(xq, sx, qw, sw, bd, "i8", "i8", 4)
        side.synchronize()
        assert ops._splitk_ws[key] is not ws_before and any(t is ws_before for t in ops._splitk_retired)
        assert _same(big, ops.linear_i8(xq, sx, qw, sw, bd))
    torch.cuda.synchronize()
    ref = O.linear_int8(x, *O.weight_quant_int8(w), b)["out"]
    assert _same(eager0, ref)
    for seed in (79, 80, 81):
        x2, _, _ = O.make_inputs(m, k, n, seed=seed)
        want = run(x2.to(dev))
        torch.cuda.synchronize()
        static_x.copy_(x2.to(dev))
        graph.replay()
        torch.cuda.synchronize()
        assert _same(static_out, want), f"replay with seed {seed} differs from eager"


@pytest.mark.parametrize("m,n,k,order,tail", [(700, 2304, 1024, 2002, 3000), (4100, 4352, 256, 2001, 3002), (4725, 5120, 256, 2001, 3000)])
@pytest.mark.parametrize("fp8", [False, True])
def test_captured_graph_of_the_256_tile_kernels_replays_match_eager(fp8, m, n, k, order, tail):
    """The kernels the large shapes run on (INT8 16x16x64, FP8 16x16x128; chosen by argument here because the shape
    is small), captured and replayed with new operand contents: in the banded tile order with its padding workgroups,
    and as the grids whose last round of workgroups runs in smaller pieces (289 tiles: 256 + 33 as quadrants; 380 tiles:
    256 + 124 as halves)."""
    import dax_amd.ops as ops
    from dax_amd import _capi

    g = torch.Generator().manual_seed(3)
    sx, sw = (torch.rand(m, generator=g) + 0.5).cuda(), (torch.rand(n, generator=g) * 0.01).cuda()
    b = torch.randn(n, generator=g).bfloat16().cuda()

    def operands(seed):
        gg = torch.Generator().manual_seed(seed)
        x = torch.randint(-100, 101, (m, k), dtype=torch.int8, generator=gg)
        w = torch.randint(-100, 101, (n, k), dtype=torch.int8, generator=gg)
        if fp8:   # any byte but the two NaN codes is a finite e4m3fn value
            x, w = x.view(torch.uint8), w.view(torch.uint8)
            x = torch.where((x & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), x)
            w = torch.where((w & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), w)
        return x.cuda(), w.cuda()

    fn = ops.linear_e4m3 if fp8 else ops.linear_i8
    try:
        _capi.debug_select_gemm(8)
        _capi.debug_select_gemm(order)
        _capi.debug_select_gemm(tail)
        static_x, static_w = operands(0)
        fn(static_x, sx, static_w, sw, b)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_out = fn(static_x, sx, static_w, sw, b)
        for seed in (1, 2, 3):
            x, w = operands(seed)
            eager = fn(x, sx, w, sw, b)
            torch.cuda.synchronize()
            static_x.copy_(x)
            static_w.copy_(w)
            graph.replay()
            torch.cuda.synchronize()
            assert _same(static_out, eager), f"replay with seed {seed} differs from eager"
    finally:
        _capi.debug_select_gemm(0)
        _capi.debug_select_gemm(2000)
        _capi.debug_select_gemm(3000)


_FIRST_LAUNCH_IN_CAPTURE = r"""
import sys
import torch
from torch import nn
sys.path.insert(0, sys.argv[1])
from dax_amd.quant.quantization import quantize_dynamic
from dax_amd.quant.quantization.qconfig import (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig,
                                                get_dynamic_int8_per_token_act_per_channel_weight_qconfig)
for fp8 in (False, True):
    torch.manual_seed(0)
    model = nn.Sequential(nn.Linear(640, 1024), nn.GELU(approximate="tanh"), nn.Linear(1024, 640)).bfloat16().cuda()
    cfg = (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(activation_dtype=torch.float8_e4m3fn)
           if fp8 else get_dynamic_int8_per_token_act_per_channel_weight_qconfig())
    quantize_dynamic(model, {"": cfg})
    x = torch.randn(2, 520, 640, device="cuda").bfloat16()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):      # no forward has run yet in this process
        y = model(x)
    graph.replay()
    torch.cuda.synchronize()
    captured = y.clone()
    eager = model(x)
    torch.cuda.synchronize()
    assert torch.equal(captured.view(torch.int16), eager.view(torch.int16)), "fp8" if fp8 else "int8"
print("first-launch-in-capture ok")
"""


def test_first_forward_of_a_process_inside_a_capture():
    """The library prepares its kernels (daxq_init) when a device is first used, so nothing has to be launched
    before a capture: a fresh process captures its very first forward and the replay equals eager."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", _FIRST_LAUNCH_IN_CAPTURE, root], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0 and "first-launch-in-capture ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]


def test_init_is_idempotent():
    from dax_amd import _capi

    for _ in range(3):
        assert _capi.lib().daxq_init() == 0, _capi.last_error()
