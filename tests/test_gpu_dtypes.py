"""GPU parity for the wider surface of the reference's quantised linear: the dynamic-quantisation entry points
themselves (dax/quant/nn/dynamic/functional.py:54-206) for every block scheme and input dtype, fp16 / fp32 modules,
e5m2 weights, the un-compiled small-shape fallback, and the error paths that must fire before any launch.
Everything goes through torch.ops.daxq -> the C ABI; the checker is the CPU oracle.
"""
import numpy as np
import pytest
import torch
from torch import nn

from oracle import daxq_oracle as O
from tests.util import bf16_bits, rel_l2

pytestmark = pytest.mark.gpu
FP8_TOL = 2e-2
TARGETS = [torch.int8, torch.float8_e4m3fn, torch.float8_e5m2]


def _bytes(q):
    return q.cpu().view(torch.uint8) if q.dtype != torch.int8 else q.cpu()


def _x(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g) * torch.logspace(-2, 2, shape[-1])
    return x.to(dtype)


# ------------------------------------------------------------------ a4: the wrappers, called directly
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(37, 392), (3, 50, 256), (2, 3, 16, 136), (5, 8)])
def test_dynamic_quantize_wrappers_per_token_and_per_tensor(dtype, shape):
    """dynamic_quantize_to_int8 / _to_fp8 on 2-d, 3-d and 4-d inputs (K a multiple of 128 or not): values, scales,
    shapes and dtypes equal to the oracle's, bit for bit."""
    from dax_amd.quant import per_tensor_symmetric, per_token_symmetric
    from dax_amd.quant.nn.dynamic.functional import dynamic_quantize_to_fp8, dynamic_quantize_to_int8

    x = _x(shape, dtype, seed=len(shape) * 100 + shape[-1])
    x.view(-1, shape[-1])[1] = 0  # a zero row: scale 2^-23
    xd = x.cuda()
    for scheme in (per_token_symmetric, per_tensor_symmetric):
        block = O.get_block_size(tuple(shape), scheme)
        for target in TARGETS:
            if target == torch.int8:
                q, s = dynamic_quantize_to_int8(xd, qscheme=scheme)
            else:
                q, s = dynamic_quantize_to_fp8(xd, qscheme=scheme, target_dtype=target)
            qo, so = O.dynamic_quantize(x, block, target)
            assert q.shape == qo.shape == x.shape and q.dtype == target
            assert s.dtype == torch.float32 and tuple(s.shape) == tuple(so.shape), (scheme, s.shape, so.shape)
            assert torch.equal(s.cpu(), so), (scheme, target, dtype)
            assert torch.equal(_bytes(q), _bytes(qo)), (scheme, target, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape,block", [((6, 40, 96), (6, 40, 1)), ((6, 40, 96), (1, 1, 32)), ((6, 40, 96), (1, 8, 96)),
                                         ((6, 40, 96), (2, 40, 48)), ((3, 3, 10, 10), (3, 3, 2, 10)), ((64, 256), (16, 128)),
                                         ((64, 256), (64, 1)), ((12, 8), (1, 8)), ((12, 8), (1, 2))])
def test_dynamic_quantize_func_any_block(dtype, shape, block):
    """_dynamic_quantize_func with explicit blocks: per-channel activations, last-dimension groups, 2-d tiles, blocks
    over leading dimensions (the reference's own docstring example among them)."""
    from dax_amd.quant.nn.dynamic.functional import _dynamic_quantize_func, dynamic_quantize_to_int8

    x = _x(shape, dtype, seed=sum(shape) + sum(block))
    xd = x.cuda()
    for target in TARGETS:
        qmax = 127 if target == torch.int8 else torch.finfo(target).max
        q, s = _dynamic_quantize_func(xd, list(block), target, quant_max=qmax, eps=torch.finfo(torch.float32).eps,
                                      scale_dtype=torch.float32)
        qo, so = O.dynamic_quantize(x, block, target)
        assert tuple(s.shape) == tuple(so.shape) and q.shape == x.shape and q.dtype == target
        assert torch.equal(s.cpu(), so), (target, block)
        assert torch.equal(_bytes(q), _bytes(qo)), (target, block)
    q, s = dynamic_quantize_to_int8(xd, block_size=list(block))   # block_size overrides the qscheme
    assert torch.equal(q.cpu(), O.dynamic_quantize(x, block, torch.int8)[0])


def test_dynamic_quantize_rejects_what_the_reference_rejects():
    from dax_amd.quant.nn.dynamic.functional import dynamic_quantize_to_fp8, dynamic_quantize_to_int8

    x = torch.zeros(4, 8, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(AssertionError):
        dynamic_quantize_to_int8(x, qscheme="nonsense")
    with pytest.raises(AssertionError):
        dynamic_quantize_to_int8(x.to(torch.float64), qscheme="dax.quant.per_token_symmetric")
    with pytest.raises(NotImplementedError):
        dynamic_quantize_to_fp8(x, target_dtype=torch.int8)
    with pytest.raises(AssertionError):
        dynamic_quantize_to_int8(x, block_size=[1, 3])           # 8 is not divisible by 3
    q, s = dynamic_quantize_to_int8(x[:0], qscheme="dax.quant.per_token_symmetric")   # empty input
    assert q.shape == (0, 8) and s.shape == (0, 1)


# ------------------------------------------------------------------ modules that are not bf16
def _module(k, n, dtype, seed, bias=True):
    x, w, b = O.make_inputs(8, k, n, seed=seed)
    lin = nn.Linear(k, n, bias=bias).to(dtype)
    with torch.no_grad():
        lin.weight.copy_(w.to(dtype))
        if bias:
            lin.bias.copy_(b.to(dtype))
    return nn.Sequential(lin), w.to(dtype), (b.to(dtype) if bias else None)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("m,k,n", [(300, 392, 264), (1100, 1024, 520), (20, 128, 40), (2900, 256, 3080)])
def test_int8_module_fp16_fp32_bit_exact(dtype, m, k, n):
    """out_dtype = the float weight's dtype (dax/quant/nn/dynamic/linear.py:263): scale in the input's dtype, fp32
    scaling of the exact accumulators, cast to fp16 / fp32, bias added in that dtype.  fp16 modules run the tiled
    and fp32 modules run the tiled kernels (128x128 tiles for the first two shapes, 256x256 with edge tiles for the last)."""
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    model, w, b = _module(k, n, dtype, seed=m + k)
    model.cuda()
    quantize_dynamic(model, {"": cfg()})
    lin = model[0]
    assert lin.out_dtype == dtype and lin.bias.dtype == dtype
    qw, sw = O.weight_quant_int8(w)
    assert torch.equal(lin.qweight.cpu(), qw) and torch.equal(lin.weight_scale.cpu(), sw)
    x = _x((m, k), dtype, seed=m)
    y = model(x.cuda())
    ref = O.linear_int8(x, qw, sw, b)["out"]
    assert y.dtype == dtype
    assert torch.equal(y.cpu(), ref), f"{(y.cpu() != ref).sum().item()} of {ref.numel()} outputs differ"
    # a bf16 input into this module: quantised by the bf16 rule, output still in the module's dtype
    xb = x.bfloat16()
    yb = model(xb.cuda())
    xq, sx = O.act_quant_int8(xb)
    refb = O.epilogue_int8(O.int_mm(xq, qw), sx, sw, b, dtype)
    assert yb.dtype == dtype and torch.equal(yb.cpu(), refb)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("variant,m,n,k", [(8, 700, 520, 256), (11, 300, 392, 384), (8, 4100, 4352, 128), (0, 130, 264, 128),
                                           (8, 4725, 5120, 128)])
def test_int8_fp16_fp32_outputs_of_the_tiled_kernels(variant, m, n, k, dtype):
    """fp16 / fp32 outputs straight from the kernels on 16x16 MFMAs, named by argument, with and without bias, edge
    tiles included; 289 tiles with the tiles left over after one round forced into quadrants, 380
    tiles with the 124 left over as 256x128 halves (all of them write the type).  Values beyond the fp16 range become infinities, as the reference's cast makes them."""
    import dax_amd.ops as ops
    from dax_amd import _capi

    g = torch.Generator().manual_seed(variant + m)
    xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, generator=g)
    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g)
    sx, sw = torch.rand(m, generator=g) + 0.5, torch.rand(n, generator=g) * 0.01
    sx[0] = 3.0e4                                   # a row that overflows fp16
    b = torch.randn(n, generator=g).to(dtype)
    acc = O.int_mm(xq, wq)
    try:
        _capi.debug_select_gemm(variant)
        _capi.debug_select_gemm(2001)
        _capi.debug_select_gemm(3002)
        for bias in (b, None):
            out = ops.linear_w8a8(xq.cuda(), sx.cuda(), wq.cuda(), sw.cuda(), bias.cuda() if bias is not None else None, "i8", "i8", dtype)
            ref = O.epilogue_int8(acc, sx.view(-1, 1), sw.view(1, -1), bias, dtype)
            assert out.dtype == dtype and (dtype == torch.float32 or torch.isinf(ref[0]).any())
            bits = torch.int16 if dtype == torch.float16 else torch.int32
            assert torch.equal(out.cpu().view(bits), ref.view(bits)), f"{(out.cpu().view(bits) != ref.view(bits)).sum().item()} outputs differ"
    finally:
        for v in (0, 2000, 3000):
            _capi.debug_select_gemm(v)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("x_fmt,w_fmt", [("e4m3", "e4m3"), ("e5m2", "e4m3"), ("e4m3", "e5m2")])
@pytest.mark.parametrize("variant,m,n,k", [(8, 700, 520, 640), (11, 300, 392, 384), (8, 4100, 4352, 256), (0, 130, 264, 128),
                                           (8, 4725, 5120, 256)])
def test_fp8_fp16_fp32_outputs_of_the_tiled_kernels(variant, m, n, k, dtype, x_fmt, w_fmt):
    """fp16 / fp32 outputs of FP8 operands (what a per-tensor FP8 module that is not bf16 asks for) from the kernel on
    16x16x128 MFMAs, on both tile sizes, with and without bias, and with the last round cut into smaller pieces
    (quadrants, or 256x128 halves in the last shape):
    out = T(acc * sx * sw + bias) with one rounding, against the oracle's scaled matmul at 3e-3 relative L2, and
    against the same kernel's bf16 launch (its accumulators are the same, so its fp32 result rounded to bf16 must
    equal the bf16 output bit for bit)."""
    import dax_amd.ops as ops
    from dax_amd import _capi

    fdt = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}
    g = torch.Generator().manual_seed(variant + m + len(x_fmt))
    xf = (torch.randn(m, k, generator=g) * 3).to(fdt[x_fmt])
    wf = (torch.randn(n, k, generator=g) * 0.5).to(fdt[w_fmt])
    sx, sw = torch.rand(m, generator=g) * 0.1 + 0.01, torch.rand(n, generator=g) * 0.01 + 1e-3
    b = torch.randn(n, generator=g).to(dtype)
    try:
        _capi.debug_select_gemm(variant)
        _capi.debug_select_gemm(2001)
        _capi.debug_select_gemm(3002)
        for bias in (b, None):
            bd = bias.cuda() if bias is not None else None
            out = ops.linear_w8a8(xf.view(torch.uint8).cuda(), sx.cuda(), wf.view(torch.uint8).cuda(), sw.cuda(), bd, x_fmt, w_fmt, dtype)
            ref = O.scaled_mm_fp32(xf, wf, sx, sw, bias, dtype)
            assert out.dtype == dtype and rel_l2(out, ref) < 3e-3
            if dtype == torch.float32:
                outb = ops.linear_w8a8(xf.view(torch.uint8).cuda(), sx.cuda(), wf.view(torch.uint8).cuda(), sw.cuda(),
                                       bd.bfloat16() if bd is not None else None, x_fmt, w_fmt, torch.bfloat16)
                if bias is None:
                    assert torch.equal(out.bfloat16(), outb)
    finally:
        for v in (0, 2000, 3000):
            _capi.debug_select_gemm(v)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("per_tensor", [False, True])
def test_fp8_module_fp16_fp32(dtype, per_tensor):
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization import qconfig as Q

    m, k, n = 520, 640, 384
    model, w, b = _module(k, n, dtype, seed=9)
    model.cuda()
    cfg = (Q.get_default_dynamic_fp8_qconfig(activation_dtype=torch.float8_e4m3fn) if per_tensor else
           Q.get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(activation_dtype=torch.float8_e4m3fn))
    quantize_dynamic(model, {"": cfg})
    lin = model[0]
    assert lin.bias.dtype == (dtype if per_tensor else torch.bfloat16)
    act = lin.input_dtype
    if per_tensor:
        sw = O.weight_scale_per_tensor(w, O.E4M3_QMAX)
        qw = O.quantize_to_fp8(w, sw)
    else:
        qw, sw = O.weight_quant_e4m3(w)
    assert torch.equal(lin.qweight.cpu().view(torch.uint8), qw.view(torch.uint8))
    assert torch.equal(lin.weight_scale.cpu().reshape(-1), sw.reshape(-1))
    x = _x((m, k), dtype, seed=10)
    y = model(x.cuda())
    ref = O.linear_fp8(x, qw, sw, b, act_dtype=act, per_tensor=per_tensor)["out"]
    assert y.dtype == dtype and rel_l2(y, ref) < 3e-3
    if not per_tensor:   # rounded to bf16 first, then cast: every output is a bf16 value
        assert torch.equal(y, y.bfloat16().to(dtype))


# ------------------------------------------------------------------ e5m2 weights
@pytest.mark.parametrize("variant", [0, 5, 8, 11, 2])
@pytest.mark.parametrize("x_e5m2", [False, True])
def test_e5m2_weights_accumulators_and_outputs(variant, x_e5m2):
    """e5m2 weight bytes through every FP8 kernel: accumulators against the exact float64 sum of the decoded products
    (a wrong format select is off by orders of magnitude), outputs against the oracle."""
    import dax_amd.ops as ops
    from dax_amd import _capi

    m, n, k = 600, 520, 512
    act = torch.float8_e5m2 if x_e5m2 else torch.float8_e4m3fn
    x, w, b = O.make_inputs(m, k, n, seed=31 + variant)
    qw, sw = O.weight_quant_fp8(w, torch.float8_e5m2)
    ref = O.linear_fp8(x, qw, sw, b, act_dtype=act)
    xq, sx = (ops.act_quant_e5m2 if x_e5m2 else ops.act_quant_e4m3)(x.cuda())
    assert torch.equal(xq[:, :k].cpu(), ref["xq"].view(torch.uint8))
    _capi.debug_select_gemm(variant)
    try:
        out, acc = ops.linear_w8a8_acc(xq, sx, qw.view(torch.uint8).cuda(), sw.view(-1).cuda(), b.cuda(),
                                       "e5m2" if x_e5m2 else "e4m3", "e5m2", torch.bfloat16)
    finally:
        _capi.debug_select_gemm(0)
    want = ref["xq"].double() @ qw.double().t()
    bound = ref["xq"].double().abs() @ qw.double().abs().t()
    err = ((acc.cpu().double() - want).abs() / bound.clamp_min(1e-30)).max().item()
    # relative to the sum of the products' magnitudes.  e4m3fn x e4m3fn stays below 2e-5; e5m2 weights spread the
    # products of one instruction over more binades, and the MFMA aligns the 64 products of an instruction in an adder
    # of limited width before the fp32 accumulate, so the bound is wider (measured 4e-5 to 6e-5).  A wrong format
    # select is off by orders of magnitude.
    assert err < 1.5e-4, err
    assert rel_l2(out, ref["out"]) < 3e-3


# ------------------------------------------------------------------ small shapes: the un-compiled reference's float matmul
def test_small_shape_fallback_switch_and_deviation():
    """Default: every shape is quantised, which is what the reference does as shipped (its forward is compiled, and
    `not is_compiling()` guards the fallback, dax/quant/nn/dynamic/linear.py:143,195).  With the switch on, M <= 16 (or
    K / N not multiples of 8) runs the float matmul on the de-quantised weight.  The two differ by the activation
    quantisation error, bounded here."""
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    k, n = 512, 256
    model, w, b = _module(k, n, torch.bfloat16, seed=77)
    model.cuda()
    quantize_dynamic(model, {"": cfg()})
    lin = model[0]
    qw, sw = O.weight_quant_int8(w)
    for m in (1, 16, 17):
        x, _, _ = O.make_inputs(m, k, 8, seed=m)
        quantised = O.linear_int8(x, qw, sw, b)["out"]
        y = model(x.cuda())
        np.testing.assert_array_equal(bf16_bits(y), bf16_bits(quantised))           # default: quantised at every M
        lin.uncompiled_small_shape_fallback = True
        try:
            yf = model(x.cuda())
        finally:
            del lin.uncompiled_small_shape_fallback
        if O.takes_float_fallback(m, k, n):
            ref = O.linear_int8_float_fallback(x, qw, sw, b)
            assert rel_l2(yf, ref) < 4e-3                                             # float matmul: summation order
            dev_ = rel_l2(yf, quantised)
            assert 1e-4 < dev_ < 5e-2, dev_                                           # the documented deviation
        else:
            np.testing.assert_array_equal(bf16_bits(yf), bf16_bits(quantised))
    assert QLinear.uncompiled_small_shape_fallback is False


# ------------------------------------------------------------------ errors that must fire before any launch
def test_device_mismatch_raises_before_any_launch():
    """A quantised module left on the CPU and called with a device tensor (the reference's example quantises before
    pipe.to(device)): an exception, never a kernel launched on a host pointer."""
    import dax_amd.ops as ops
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.qscheme import per_channel_symmetric as ch, per_token_symmetric as tok

    lin = QLinear(256, 128, True, None, torch.int8, torch.int8, torch.bfloat16, ch, tok)   # on the CPU
    x = torch.zeros(32, 256, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="same device"):
        lin(x)
    xq = torch.zeros(32, 256, dtype=torch.int8, device="cuda")
    ones = torch.ones(32, device="cuda")
    wq_cpu, sw_cpu = torch.zeros(128, 256, dtype=torch.int8), torch.ones(128)
    with pytest.raises(ValueError, match="same device"):
        ops.linear_i8(xq, ones, wq_cpu, sw_cpu.cuda(), None)
    with pytest.raises(ValueError, match="same device"):
        ops.linear_i8(xq, ones, wq_cpu.cuda(), sw_cpu, None)
    with pytest.raises(ValueError, match="same device"):
        ops.linear_i8(xq, ones.cpu(), wq_cpu.cuda(), sw_cpu.cuda(), None)
    with pytest.raises(ValueError, match="same device"):
        ops.linear_i8(xq, ones, wq_cpu.cuda(), sw_cpu.cuda(), torch.zeros(128, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="same device"):
        ops.dynamic_linear_i8(x, wq_cpu, sw_cpu.cuda(), None)
    with pytest.raises(ValueError, match="same device"):
        ops.scale_from_minmax(torch.zeros(4, device="cuda"), torch.zeros(4), 127.0)
    with pytest.raises(ValueError, match="same device"):
        ops.tensor_scale(torch.zeros(4, device="cuda"), torch.zeros(4), 127.0, 1, 4)
    torch.cuda.synchronize()   # nothing faulted


def test_derived_operands_capture_then_eager_then_replay():
    """K = 392 (zero-padded weight copy) and a per-tensor weight scale (written out per channel): both derived
    operands exist before the first forward, so a first forward inside a capture leaves nothing behind that a later
    eager call would read before a replay has filled it."""
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_default_dynamic_int8_qconfig as cfg

    k, n, m = 392, 264, 300
    model, w, b = _module(k, n, torch.bfloat16, seed=5)
    model.cuda()
    quantize_dynamic(model, {"": cfg()})
    lin = model[0]
    assert lin._packed is not None and lin._sw_vec is not None      # built at conversion
    x, _, _ = O.make_inputs(m, k, 8, seed=6)
    xd = x.cuda()
    ref = O.linear_int8_schemes(x, w, b, True, True)["out"]
    lin._packed = lin._sw_vec = None                                 # the worst case: nothing cached when the capture starts
    static_x = xd.clone()
    g = torch.cuda.CUDAGraph()
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        with torch.cuda.graph(g, stream=s):
            static_y = model(static_x)
    torch.cuda.current_stream().wait_stream(s)
    assert lin._packed is None and lin._sw_vec is None               # nothing recorded was kept
    y_eager = model(xd)                                              # eager call BEFORE any replay
    np.testing.assert_array_equal(bf16_bits(y_eager), bf16_bits(ref))
    for _ in range(3):
        g.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bf16_bits(static_y), bf16_bits(ref))
        np.testing.assert_array_equal(bf16_bits(model(xd)), bf16_bits(ref))


def test_minmax_observer_with_infinite_calibration_data():
    """Only the untouched state (min = +inf, max = -inf) counts as unobserved; a real infinity in the data gives an
    infinite scale, as the reference's check does (dax/quant/quantization/observer.py:116-120)."""
    from dax_amd.quant.quantization.observer import MinMaxObserver

    obs = MinMaxObserver(dtype=torch.float8_e4m3fn).cuda()
    assert obs.calculate_qparams() is None
    x = torch.randn(8, 64).bfloat16()
    x[3, 5] = float("inf")
    obs(x.cuda())
    s = obs.calculate_qparams()
    assert s is not None and torch.isinf(s).all()
    obs.reset_min_max_vals()
    assert obs.calculate_qparams() is None
    obs(torch.ones(4, 64).bfloat16().cuda() * 3)
    assert float(obs.calculate_qparams()) == float(O.weight_scale_per_tensor(torch.ones(1, 1) * 3, O.E4M3_QMAX))
