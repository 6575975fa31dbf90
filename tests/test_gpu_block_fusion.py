"""Block-level fusion on a stand-in Wan transformer: shared quantisation is bit-identical, the fused
producers stay within the floating-point tolerance of the unfused quantised model."""
import copy

import pytest
import torch

from tests.util import rel_l2
from tests.wan_replica import Transformer

pytestmark = pytest.mark.gpu


def _model(fp8=False, cross_attn_norm=True, seed=0):
    from dax_amd.adapters.wan import quantize_transformer

    torch.manual_seed(seed)
    model = Transformer(cross_attn_norm=cross_attn_norm).to(torch.bfloat16).to("cuda")
    quantize_transformer(model, fp8=fp8)
    return model


def _inputs(model, batch=2, seq=320, text=48):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(batch, seq, model.dim, generator=g).bfloat16().cuda()
    x[..., ::37] *= 10
    ctx = torch.randn(batch, text, model.dim, generator=g).bfloat16().cuda()
    t = torch.randn(batch, model.dim, generator=g).bfloat16().cuda()
    return x, ctx, t


def test_share_input_quant_and_fuse_linears_are_bit_identical():
    from dax_amd.adapters.wan import fuse_linears, share_input_quant

    model = _model()
    attn = model.blocks[0].attn1
    x = _inputs(model)[0]
    want = [attn.to_q(x), attn.to_k(x), attn.to_v(x)]
    fused = fuse_linears([attn.to_q, attn.to_k, attn.to_v])
    got = fused(x)
    assert torch.equal(got, torch.cat(want, -1))
    calls = []
    orig = type(attn.to_q).quantize_activation

    def counting(self, inp):
        calls.append(1)
        return orig(self, inp)

    type(attn.to_q).quantize_activation = counting
    try:
        cache = share_input_quant([attn.to_q, attn.to_k, attn.to_v])
        again = [attn.to_q(x), attn.to_k(x), attn.to_v(x)]
        assert len(calls) == 1                                   # one quantisation for the three linears
        assert all(torch.equal(a, b) for a, b in zip(again, want))
        x.add_(1)                                                # in-place change: must not reuse the stale form
        attn.to_q(x)
        assert len(calls) == 2
        y = x.clone()                                            # equal contents, another tensor: a miss
        attn.to_k(y)
        assert len(calls) == 3
        del y
        z = torch.empty_like(x).copy_(x).mul_(2)                 # may reuse the freed address of y
        out_z = attn.to_v(z)
        cache.clear()
        type(attn.to_q).quantize_activation = orig
        assert torch.equal(out_z, attn.to_v(z))                  # not the stale quantised form of y
    finally:
        type(attn.to_q).quantize_activation = orig


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("cross_attn_norm", [True, False])
def test_fused_blocks_match_the_unfused_quantised_model(fp8, cross_attn_norm):
    from dax_amd.adapters.wan import fuse_transformer_blocks
    from dax_amd.quant.nn.dynamic import Linear

    model = _model(fp8, cross_attn_norm)
    x, ctx, t = _inputs(model)
    with torch.no_grad():
        ref = model(x, ctx, t)
    keys = list(model.state_dict().keys())
    fused = copy.deepcopy(model)
    assert fuse_transformer_blocks(fused) == len(fused.blocks)
    assert fuse_transformer_blocks(fused) == 0                    # idempotent
    assert list(fused.state_dict().keys()) == keys                # checkpoints stay interchangeable
    assert isinstance(fused.blocks[0].ffn.net[2], Linear)
    with torch.no_grad():
        out = fused(x, ctx, t)
    assert out.shape == ref.shape and torch.isfinite(out.float()).all()
    # the fused kernels round LayerNorm / GELU results like an fp32 evaluation does, the unfused model goes
    # through torch's kernels: single int8 / fp8 steps differ, nothing more
    assert rel_l2(out, ref) < (4e-2 if fp8 else 2e-2), rel_l2(out, ref)


def test_unquantised_blocks_are_left_alone():
    from dax_amd.adapters.wan import fuse_transformer_blocks

    model = Transformer().to(torch.bfloat16).to("cuda")
    assert fuse_transformer_blocks(model) == 0


@pytest.mark.parametrize("fused", [False, True])
@pytest.mark.parametrize("fp8", [False, True])
def test_quantised_transformer_under_torch_compile(fp8, fused):
    """The reference's deployment: the whole transformer with swapped linears inside torch.compile
    (dax/adapters/wan/functional.py:33-36).  The code generator re-fuses the fp32 LayerNorm / modulation / attention
    code around the daxq ops, so the comparison with eager is a tolerance, not bit equality."""
    pytest.importorskip("triton")
    model = _model(fp8)
    if fused:  # the explicit producer + quantiser fusions trace as well
        from dax_amd.adapters.wan import fuse_transformer_blocks

        fuse_transformer_blocks(model)
    x, ctx, t = _inputs(model)
    with torch.no_grad():
        ref = model(x, ctx, t)
        out = torch.compile(model)(x, ctx, t)
    assert out.shape == ref.shape and out.dtype == ref.dtype
    assert rel_l2(out, ref) < 2e-2
