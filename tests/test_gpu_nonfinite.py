"""Non-finite values.  The reference's scale recipe is built from torch reductions and clamps that carry a NaN
through (abs().amax(), clamp(min=eps): dax/quant/nn/dynamic/functional.py:124-127; aminmax / torch.max:
dax/quant/quantization/observer.py:97-134, 200-214), so a NaN or an infinity in a token makes that token's
scale NaN / inf and its whole output row non-finite, and leaves every other row alone.  The kernels must do the
same: a poisoned row may not come out as finite numbers.
"""
import numpy as np
import pytest
import torch

from oracle import daxq_oracle as O
from tests.util import bf16_bits

pytestmark = pytest.mark.gpu

BAD = {3: float("inf"), 5: float("nan"), 9: float("-inf")}


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import dax_amd.ops as ops

    return ops


def _poisoned(m, k, seed):
    g = torch.Generator("cpu").manual_seed(seed)
    x = torch.randn(m, k, generator=g).bfloat16()
    bad = x.clone()
    for row, val in BAD.items():
        bad[row, (row * 37) % k] = val
    return x, bad


def _same_scale(got, want):
    np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32) & 0x7fc00000 == 0x7fc00000,
                                  torch.isnan(want).numpy())           # NaN where the oracle has NaN
    ok = ~torch.isnan(want)
    np.testing.assert_array_equal(got.cpu()[ok].numpy(), want[ok].numpy())   # inf and finite values bit for bit


@pytest.mark.parametrize("variant", [0, 8])   # 8: the kernels of the large shapes (16x16 MFMA forms)
@pytest.mark.parametrize("fmt", ["i8", "e4m3", "e5m2"])
def test_poisoned_tokens_get_the_oracles_scale_and_a_nonfinite_row(ops, fmt, variant, request):
    from dax_amd import _capi

    _capi.debug_select_gemm(variant)
    request.addfinalizer(lambda: _capi.debug_select_gemm(0))
    m, k, n = 300, 512, 384
    x, bad = _poisoned(m, k, seed=1)
    g = torch.Generator("cpu").manual_seed(2)
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16().cuda()
    b = (torch.randn(n, generator=g) * 0.01).bfloat16().cuda()
    fp8 = fmt != "i8"
    lo, hi = ops.row_minmax(w)
    sw = ops.scale_from_minmax(lo, hi, 448.0 if fp8 else 127.0)
    qw = (ops.quantize_rows_e4m3 if fp8 else ops.quantize_rows_i8)(w, sw, True)
    quant = getattr(ops, "act_quant_" + fmt)
    linear = {"i8": ops.linear_i8, "e4m3": ops.linear_e4m3, "e5m2": ops.linear_e5m2_e4m3}[fmt]
    qmax = {"i8": 127.0, "e4m3": O.E4M3_QMAX, "e5m2": O.E5M2_QMAX}[fmt]

    xq, sx = quant(x.cuda())
    clean = linear(xq, sx, qw, sw, b)
    xq2, sx2 = quant(bad.cuda())
    out = linear(xq2, sx2, qw, sw, b)
    torch.cuda.synchronize()
    _same_scale(sx2, O.act_scale(bad, qmax).view(-1))
    rows = sorted(BAD)
    assert not bool(torch.isfinite(out[rows].float()).any()), "a poisoned token produced finite outputs"
    keep = [i for i in range(m) if i not in BAD]
    np.testing.assert_array_equal(bf16_bits(out[keep]), bf16_bits(clean[keep]))


@pytest.mark.parametrize("fmt", ["i8", "e4m3"])
def test_poisoned_tokens_through_the_fused_producers(ops, fmt):
    m, k = 64, 1024
    _, bad = _poisoned(m, k, seed=3)
    q, s, y = getattr(ops, "gelu_tanh_act_quant_" + fmt)(bad.cuda(), True)
    q2, s2, y2 = getattr(ops, "layernorm_act_quant_" + fmt)(bad.cuda(), None, None, m, 1e-6, True)
    torch.cuda.synchronize()
    # GELU: +inf -> +inf, -inf -> -0 * ... = NaN or 0 depending on the form; NaN -> NaN.  The scale follows the bf16 result.
    want = O.act_scale(y.cpu(), 127.0 if fmt == "i8" else O.E4M3_QMAX).view(-1)
    _same_scale(s, want)
    assert bool(torch.isnan(s[5])) and not bool(torch.isfinite(s[3]))
    # LayerNorm: a non-finite element makes mean and variance non-finite, the whole row NaN
    for row in BAD:
        assert bool(torch.isnan(y2[row].float()).all()) and bool(torch.isnan(s2[row]))
    keep = [i for i in range(m) if i not in BAD]
    assert bool(torch.isfinite(s2[keep]).all()) and bool(torch.isfinite(y2[keep].float()).all())


def test_poisoned_statistics_of_weights_and_whole_tensors(ops):
    n, k = 40, 256
    _, bad = _poisoned(n, k, seed=4)
    lo, hi = ops.row_minmax(bad.cuda())
    sw = ops.scale_from_minmax(lo, hi, 127.0)
    torch.cuda.synchronize()
    want = O.weight_scale(bad, 127.0).view(-1)
    _same_scale(sw, want)
    # per tensor: one NaN anywhere makes the scale NaN (amax() / aminmax carry it)
    s1, _ = ops.tensor_scale(lo, hi, 448.0, True, 4)
    assert bool(torch.isnan(s1).all())
    mn = torch.tensor([-1.0], device="cuda")
    mx = torch.tensor([1.0], device="cuda")
    ops.tensor_minmax_update(lo, hi, mn, mx)
    assert bool(torch.isnan(mn).all()) and bool(torch.isnan(mx).all())
    # without the NaN row: infinities remain and give an infinite scale
    rows = [i for i in range(n) if i != 5]
    s2, _ = ops.tensor_scale(lo[rows].contiguous(), hi[rows].contiguous(), 448.0, True, 4)
    assert bool(torch.isinf(s2).all())


def test_leaf_quantiser_with_a_given_scale_keeps_nan(ops):
    """quantize_to_fp8 with a scale from the caller (static activations, weights): (x / s).clamp(-qmax, qmax).to(fp8),
    dax/quant/nn/quantized/functional.py:11-13 -- the clamp passes a NaN on and the cast gives the format's NaN byte;
    an infinity is clamped to the largest finite value."""
    m, k = 16, 256
    _, bad = _poisoned(m, k, seed=5)
    scale = torch.full((m,), 0.5, dtype=torch.float32)
    for fmt, dtype in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        got = getattr(ops, "quantize_rows_" + fmt)(bad.cuda(), scale.cuda(), False).cpu()
        want = O.quantize_to_fp8(bad, scale.view(-1, 1), dtype).view(torch.uint8)
        nan_byte = torch.isnan(want.view(dtype).float())
        assert int(nan_byte.sum()) == 1
        np.testing.assert_array_equal(torch.isnan(got.view(dtype).float()).numpy(), nan_byte.numpy())
        np.testing.assert_array_equal(got[~nan_byte].numpy(), want[~nan_byte].numpy())
