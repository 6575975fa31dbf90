"""On-disk format and caller integration, checked against the CPU oracle (not against this package's own
unfused model): a saved quantised model loaded straight onto the device, and the fused / unfused quantised
stand-in transformer against the same model evaluated on the CPU with every quantised linear replaced by the
oracle's forward.
"""
import copy

import numpy as np
import pytest
import torch
from torch import nn

from oracle import daxq_oracle as O
from tests.util import bf16_bits, rel_l2
from tests.wan_replica import Transformer

pytestmark = pytest.mark.gpu
FP8_TOL = 2e-2


class OracleLinear(nn.Module):
    """The reference's dynamic quantised linear as the CPU oracle computes it: conversion and forward."""

    def __init__(self, lin: nn.Linear, fp8: bool):
        super().__init__()
        w = lin.weight.detach()
        self.b = None if lin.bias is None else lin.bias.detach()
        self.fp8 = fp8
        self.qw, self.sw = (O.weight_quant_e4m3 if fp8 else O.weight_quant_int8)(w)

    def forward(self, x):
        if self.fp8:
            return O.linear_fp8(x, self.qw, self.sw, self.b)["out"]
        return O.linear_int8(x, self.qw, self.sw, self.b)["out"]


def oracle_model(float_model: nn.Module, fp8: bool) -> nn.Module:
    """CPU copy of the float model in which every nn.Linear that the adapter quantises (everything outside
    condition_embedder / proj_out, dax/adapters/wan/transformer_adapter.py:227-234) runs the oracle."""
    m = copy.deepcopy(float_model).cpu()

    def walk(mod, prefix):
        for name, child in list(mod.named_children()):
            path = f"{prefix}.{name}" if prefix else name
            if path in ("condition_embedder", "proj_out"):
                continue
            if type(child) is nn.Linear:
                mod._modules[name] = OracleLinear(child, fp8)
            else:
                walk(child, path)
    walk(m, "")
    return m


def _float_model(seed=0, **kw):
    torch.manual_seed(seed)
    return Transformer(**kw).to(torch.bfloat16)


def _inputs(model, batch=2, seq=320, text=48):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(batch, seq, model.dim, generator=g).bfloat16()
    x[..., ::37] *= 10
    ctx = torch.randn(batch, text, model.dim, generator=g).bfloat16()
    t = torch.randn(batch, model.dim, generator=g).bfloat16()
    return x, ctx, t


# ------------------------------------------------------------------ f3: file -> device -> forward
@pytest.mark.parametrize("fp8", [False, True])
def test_saved_model_loaded_on_the_device_matches_the_oracle(tmp_path, fp8):
    """save_quantized -> load_quantized(meta skeleton, device="cuda") -> forward of every quantised linear against
    the oracle run on the ORIGINAL float weights: INT8 bit for bit, FP8 within 2e-2."""
    from dax_amd.adapters.wan import quantize_transformer
    from dax_amd.quant.checkpoint import load_quantized, save_quantized
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.quantization import qconfig as Q

    src = _float_model(3)
    ref = oracle_model(src, fp8)
    q = copy.deepcopy(src).cuda()
    quantize_transformer(q, fp8=fp8)
    path = str(tmp_path / "wan_standin.safetensors")
    save_quantized(q, path)
    del q
    with torch.device("meta"):
        skel = Transformer().to(torch.bfloat16)
    cfg = (Q.get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(activation_dtype=torch.float8_e4m3fn) if fp8
           else Q.get_dynamic_int8_per_token_act_per_channel_weight_qconfig())
    loaded = load_quantized(skel, path, {"": cfg, "condition_embedder": None, "proj_out": None}, device="cuda")
    assert not any(p.device.type == "meta" for p in loaded.parameters())
    g = torch.Generator().manual_seed(5)
    checked = 0
    for name, mod in loaded.named_modules():
        if not isinstance(mod, QLinear):
            continue
        oracle_lin = ref.get_submodule(name)
        assert isinstance(oracle_lin, OracleLinear)
        assert torch.equal(mod.qweight.cpu().view(torch.uint8), oracle_lin.qw.view(torch.uint8)), name
        assert torch.equal(mod.weight_scale.cpu(), oracle_lin.sw), name
        x = (torch.randn(3, 67, mod.in_features, generator=g) * 2).bfloat16()
        y = mod(x.cuda())
        want = oracle_lin(x)
        if fp8:
            assert rel_l2(y, want) < FP8_TOL, name
        else:
            np.testing.assert_array_equal(bf16_bits(y), bf16_bits(want), err_msg=name)
        checked += 1
    assert checked == 2 * 10                                    # 2 blocks x 10 quantised linears
    assert type(loaded.proj_out) is nn.Linear and type(loaded.condition_embedder[0]) is nn.Linear


def test_loaded_module_with_padded_k_and_per_tensor_scale(tmp_path):
    """K = 392 (the GEMM reads a zero-padded copy) and per-tensor scales (written out per channel): both derived
    operands are rebuilt by the load, and the forward equals the oracle's."""
    from dax_amd.quant.checkpoint import load_quantized, save_quantized
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_default_dynamic_int8_qconfig as cfg

    k, n = 392, 264
    x, w, b = O.make_inputs(150, k, n, seed=8)
    lin = nn.Linear(k, n).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    model = nn.Sequential(lin).cuda()
    quantize_dynamic(model, {"": cfg()})
    path = str(tmp_path / "one.safetensors")
    save_quantized(model, path)
    with torch.device("meta"):
        skel = nn.Sequential(nn.Linear(k, n).bfloat16())
    loaded = load_quantized(skel, path, {"": cfg()}, device="cuda")
    assert loaded[0]._packed is not None and loaded[0]._packed[1].shape == (n, 512) and loaded[0]._sw_vec is not None
    want = O.linear_int8_schemes(x, w, b, True, True)["out"]
    np.testing.assert_array_equal(bf16_bits(loaded(x.cuda())), bf16_bits(want))


# ------------------------------------------------------------------ f4: the quantised transformer against the oracle chain
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("fused", [False, True])
def test_quantised_transformer_against_the_cpu_oracle_chain(fp8, fused):
    """The stand-in transformer with swapped linears (plain, and with the block fusions: norm + modulation +
    quantiser in one kernel, one quantisation shared by q / k / v, GELU + quantiser) against the same float model
    evaluated on the CPU with the oracle's quantised linear in place of every swapped layer.  LayerNorm, GELU,
    softmax and the float adds round differently on the two devices, so single quantised values differ by a step
    here and there: a tolerance on the block outputs, and a tighter one on the first quantised projection."""
    from dax_amd.adapters.wan import quantize_transformer

    src = _float_model(11)
    ref = oracle_model(src, fp8)
    q = copy.deepcopy(src).cuda()
    quantize_transformer(q, fp8=fp8, fuse_blocks=fused)
    x, ctx, t = _inputs(src)
    with torch.no_grad():
        want = ref(x, ctx, t)
        got = q(x.cuda(), ctx.cuda(), t.cuda())
    assert got.shape == want.shape and torch.isfinite(got.float()).all()
    r = rel_l2(got, want)
    assert r < (4e-2 if fp8 else 2e-2), r
    # first stage alone (norm1 + modulation -> quantiser -> to_q): the quantised projection's input is produced by
    # the fused kernel on one side and by torch's fp32 LayerNorm on the other
    with torch.no_grad():
        temb = ref.condition_embedder(t).unflatten(1, (6, -1))
        blk = ref.blocks[0]
        shift, scale = (blk.scale_shift_table + temb.float()).chunk(6, dim=1)[:2]
        nh = (blk.norm1(x.float()) * (1 + scale) + shift).type_as(x)
        want_q = blk.attn1.to_q(nh)
        temb_d = q.condition_embedder(t.cuda()).unflatten(1, (6, -1))
        bd = q.blocks[0]
        if fused:
            from dax_amd.adapters.wan.block_fusion import layernorm_quant

            shift_d, scale_d = (bd.scale_shift_table + temb_d.float()).chunk(6, dim=1)[:2]
            got_q = bd.attn1.to_q(layernorm_quant(x.cuda(), 1 + scale_d, shift_d, 1e-6, bd.attn1.to_q))
        else:
            shift_d, scale_d = (bd.scale_shift_table + temb_d.float()).chunk(6, dim=1)[:2]
            got_q = bd.attn1.to_q((bd.norm1(x.cuda().float()) * (1 + scale_d) + shift_d).type_as(x.cuda()))
    assert rel_l2(got_q, want_q) < (1.5e-2 if fp8 else 5e-3), rel_l2(got_q, want_q)
