"""GPU parity of the arguments and switches around the activation scale:

* ``_dynamic_quantize_func`` with the caller's quant_max / eps / scale_dtype (dax/quant/nn/dynamic/functional.py:54-148),
* the per-token scale kept in fp32 (``scale_fp32`` / ``Linear.act_scale_fp32``): what is left of the eager chain when the
  reference's forward runs under its torch.compile decorator (dax/quant/nn/dynamic/linear.py:143),
* an observer with its own floor ``eps`` (dax/quant/quantization/observer.py:19-35, :125).

Everything goes through torch.ops.daxq -> the C ABI and is compared with the CPU oracle, bit for bit (FP8 matmul outputs
within the stated 2e-2 relative L2).
"""
import numpy as np
import pytest
import torch
from torch import nn

from oracle import daxq_oracle as O
from tests.util import ALL_POS_FINITE, bf16_bits, from_bits, rel_l2

pytestmark = pytest.mark.gpu
TARGETS = [torch.int8, torch.float8_e4m3fn, torch.float8_e5m2]
QMAX = {torch.int8: 127.0, torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


def _bytes(q):
    return q.cpu().view(torch.uint8) if q.dtype != torch.int8 else q.cpu()


def _x(shape, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(*shape, generator=g) * torch.logspace(-2, 2, shape[-1])
    return x.to(dtype)


@pytest.mark.parametrize("fmt,target", [("i8", torch.int8), ("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
def test_fp32_scale_every_bf16_row_maximum(fmt, target):
    """One row per non-negative finite bf16 value as the row's abs-max: scale = max(f32(amax) / qmax, 2^-23), not rounded
    to bf16, and the row's quantised values, against the oracle."""
    import dax_amd.ops as ops

    amax = from_bits(ALL_POS_FINITE)                       # [32640]
    g = torch.Generator().manual_seed(5)
    frac = (torch.rand(amax.numel(), 16, generator=g) * 2 - 1)
    x = (amax.float().view(-1, 1) * frac).bfloat16()
    x[:, 0] = amax                                          # the row maximum itself, positive
    x[:, 1] = -amax
    q, s = getattr(ops, "act_quant_" + fmt)(x.cuda(), True)
    so = O.act_scale_fp32(x, QMAX[target])
    assert torch.equal(s.cpu().view(-1, 1), so)
    qo = O.quantize_to_int8(x, so) if target == torch.int8 else O.quantize_to_fp8(x, so, target).view(torch.uint8)
    assert torch.equal(_bytes(q[:, :16]), qo if target == torch.int8 else qo)
    eager = O.act_scale(x, QMAX[target])
    assert not torch.equal(so, eager)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(300, 520), (33, 200), (4, 5120)])
def test_fp32_scale_rows_of_every_input_type(dtype, shape):
    """Random rows (K a multiple of 8 or not: both row kernels), all three formats and input types."""
    import dax_amd.ops as ops

    x = _x(shape, dtype, seed=shape[0] + shape[1])
    x[1] = 0
    for fmt, target in (("i8", torch.int8), ("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        q, s = getattr(ops, "act_quant_" + fmt)(x.cuda(), True)
        so = O.act_scale_fp32(x, QMAX[target])
        assert torch.equal(s.cpu().view(-1, 1), so), (fmt, dtype)
        qo = O.quantize_to_int8(x, so) if target == torch.int8 else O.quantize_to_fp8(x, so, target).view(torch.uint8)
        assert torch.equal(_bytes(q[:, :shape[1]]), qo), (fmt, dtype)
        assert bool((q[:, shape[1]:] == 0).all())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("quant_max,eps", [(100.0, 1e-3), (63, 0.0078125), (300.0, 0.0), (127.0, 2.0 ** -23)])
@pytest.mark.parametrize("shape,block", [((37, 392), (1, 392)), ((6, 40, 96), (1, 1, 32)), ((6, 40, 96), (6, 40, 96)),
                                         ((6, 40, 96), (6, 40, 1)), ((64, 256), (16, 128))])
def test_dynamic_quantize_func_with_the_callers_arguments(dtype, quant_max, eps, shape, block):
    """quant_max, eps and every scale_dtype (None = the input's own) for per-token, group, per-tensor, per-channel and
    tile blocks: values, scales, scale dtype and shape equal to the oracle's."""
    from dax_amd.quant.nn.dynamic.functional import _dynamic_quantize_func

    x = _x(shape, dtype, seed=sum(shape) + sum(block) + int(quant_max))
    if eps > 0:   # (with eps = 0 a zero block divides by zero, in the reference as here, and the cast of that NaN is unspecified)
        x.view(-1, shape[-1])[0] = 0
    xd = x.cuda()
    for target in TARGETS:
        for sd in (torch.float32, torch.bfloat16, torch.float16, None):
            q, s = _dynamic_quantize_func(xd, list(block), target, quant_max=quant_max, eps=eps, scale_dtype=sd)
            qo, so = O.dynamic_quantize(x, block, target, quant_max=quant_max, eps=eps, scale_dtype=sd)
            assert s.dtype == so.dtype and tuple(s.shape) == tuple(so.shape) and q.dtype == target, (target, sd)
            assert torch.equal(s.cpu().float(), so.float()), (target, sd, block)
            assert torch.equal(_bytes(q), _bytes(qo)), (target, sd, block)


def test_dynamic_quantize_func_fp32_chain_any_block():
    """scale_fp32 through _dynamic_quantize_func for row, per-tensor and general blocks."""
    from dax_amd.quant.nn.dynamic.functional import _dynamic_quantize_func

    for shape, block in (((37, 392), (1, 392)), ((6, 40, 96), (6, 40, 96)), ((6, 40, 96), (1, 8, 96)), ((64, 256), (64, 1))):
        x = _x(shape, torch.bfloat16, seed=sum(shape))
        for target in TARGETS:
            q, s = _dynamic_quantize_func(x.cuda(), list(block), target, quant_max=QMAX[target],
                                          eps=torch.finfo(torch.float32).eps, scale_dtype=torch.float32, scale_fp32=True)
            qo, so = O.dynamic_quantize(x, block, target, fused_chain=True)
            assert torch.equal(s.cpu(), so) and torch.equal(_bytes(q), _bytes(qo)), (target, block)


def test_dynamic_quantize_func_argument_errors():
    from dax_amd.quant.nn.dynamic.functional import _dynamic_quantize_func

    x = torch.zeros(4, 8, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(TypeError):          # float(None), as in the reference (:126)
        _dynamic_quantize_func(x, [1, 8], torch.int8, quant_max=None, eps=1e-7, scale_dtype=torch.float32)
    with pytest.raises(ValueError):
        _dynamic_quantize_func(x, [1, 8], torch.int8, quant_max=0, eps=1e-7, scale_dtype=torch.float32)
    with pytest.raises(NotImplementedError):
        _dynamic_quantize_func(x, [1, 8], torch.int8, quant_max=127, eps=1e-7, scale_dtype=torch.float64)


def _swapped(k, n, w, b, kind, fp32_scale):
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig,
                                                    get_dynamic_int8_per_token_act_per_channel_weight_qconfig)

    lin = nn.Linear(k, n).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    model = nn.Sequential(lin).to("cuda")
    cfg = (get_dynamic_int8_per_token_act_per_channel_weight_qconfig() if kind == "int8" else
           get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(activation_dtype=torch.float8_e4m3fn))
    quantize_dynamic(model, {"": cfg})
    model[0].act_scale_fp32 = fp32_scale
    return model


@pytest.mark.parametrize("m,k,n", [(300, 384, 520), (4096, 1536, 1536), (5, 256, 264), (700, 200, 392)])
def test_module_with_fp32_activation_scale(m, k, n):
    """Linear.act_scale_fp32 = True: INT8 outputs bit for bit against the oracle's forward with the fp32 scale, FP8
    within tolerance; the default module still gives the eager result, and the two differ."""
    x, w, b = O.make_inputs(m, k, n, seed=m + k)
    xd = x.to("cuda")
    qw, sw = O.weight_quant_int8(w)
    for fp32_scale in (True, False):
        model = _swapped(k, n, w, b, "int8", fp32_scale)
        with torch.no_grad():
            y = model(xd)
            y3 = model(xd.view(1, m, k))
        ref = O.linear_int8(x, qw, sw, b, scale_fp32=fp32_scale)["out"]
        np.testing.assert_array_equal(bf16_bits(y), bf16_bits(ref))
        np.testing.assert_array_equal(bf16_bits(y3.view(m, n)), bf16_bits(ref))
        qa = model[0].quantize_activation(xd)
        assert torch.equal(qa.sx.cpu().view(-1, 1), (O.act_scale_fp32 if fp32_scale else O.act_scale)(x, 127.0))
    a = O.linear_int8(x, qw, sw, b, scale_fp32=True)["out"]
    e = O.linear_int8(x, qw, sw, b)["out"]
    assert not torch.equal(a, e) and rel_l2(a, e) < 1e-2
    qw8, sw8 = O.weight_quant_e4m3(w)
    model = _swapped(k, n, w, b, "fp8", True)
    with torch.no_grad():
        y = model(xd)
    r8 = O.linear_fp8(x, qw8, sw8, b, scale_fp32=True)
    assert rel_l2(y, r8["out"]) < 2e-2
    qa = model[0].quantize_activation(xd)
    assert torch.equal(qa.sx.cpu().view(-1, 1), r8["sx"]) and torch.equal(qa.xq[:, :k].cpu(), r8["xq"].view(torch.uint8))


def test_block_fusion_leaves_fp32_scale_modules_alone():
    """The fused producer kernels round the scale as the eager chain does, so a block whose projections keep the scale
    in fp32 is not rebound; fuse_linears hands the switch on."""
    from dax_amd.adapters.wan import fuse_linears, fuse_transformer_blocks, quantize_transformer
    from tests.wan_replica import Transformer

    torch.manual_seed(0)
    model = Transformer().to(torch.bfloat16).to("cuda")
    quantize_transformer(model)
    n_blocks = len(model.blocks)
    model.blocks[0].attn1.to_k.act_scale_fp32 = True
    assert fuse_transformer_blocks(model) == n_blocks - 1
    assert not getattr(model.blocks[0], "_daxq_fused", False)
    a = model.blocks[0].attn1
    a.to_q.act_scale_fp32 = a.to_v.act_scale_fp32 = True
    fused = fuse_linears([a.to_q, a.to_k, a.to_v])
    assert fused.act_scale_fp32
    x = torch.randn(3, 40, model.dim, generator=torch.Generator().manual_seed(2)).bfloat16().cuda()
    assert torch.equal(fused(x), torch.cat([a.to_q(x), a.to_k(x), a.to_v(x)], -1))
    a.to_q.act_scale_fp32 = False
    with pytest.raises(ValueError):
        fuse_linears([a.to_q, a.to_k, a.to_v])


def test_observer_with_its_own_floor():
    """PerChannelMinMaxObserver / MinMaxObserver with eps other than float32 eps: scale = max(amax / qmax, eps) in fp32."""
    from dax_amd.quant import per_channel_symmetric, per_tensor_symmetric
    from dax_amd.quant.quantization.observer import MinMaxObserver, PerChannelMinMaxObserver

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(24, 64, generator=g) * torch.logspace(-4, 0, 24).view(-1, 1)).bfloat16()
    for eps in (1e-3, 0.0, 2.0 ** -23):
        obs = PerChannelMinMaxObserver(dtype=torch.int8, qscheme=per_channel_symmetric, eps=eps).to("cuda")
        obs(w.cuda())
        got = obs.calculate_qparams().cpu()
        wf = w.float()
        want = torch.max(torch.max(-wf.amin(1), wf.amax(1)) / 127.0, torch.tensor([eps]))
        assert torch.equal(got.view(-1), want)
        obs1 = MinMaxObserver(dtype=torch.float8_e4m3fn, qscheme=per_tensor_symmetric, eps=eps).to("cuda")
        obs1(w.cuda())
        want1 = torch.max(wf.abs().max() / 448.0, torch.tensor([eps]))
        assert torch.equal(obs1.calculate_qparams().cpu().view(-1), want1.view(-1))
