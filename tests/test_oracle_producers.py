"""Pins for the oracle's producer functions (LayerNorm + multiply-add, GELU-tanh).

These are floating-point functions: the pins are float64 evaluations of the textbook
formulas, special rows, and -- for GELU, a function of one bf16 value -- every input.
"""
import math

import numpy as np
import torch

from oracle import daxq_oracle as O


def _bf16_ulps(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """distance in bf16 steps between two bf16 tensors (sign-magnitude ordering)"""
    ia = a.view(torch.int16).to(torch.int32)
    ib = b.view(torch.int16).to(torch.int32)
    ia = torch.where(ia < 0, -(ia & 0x7fff), ia)
    ib = torch.where(ib < 0, -(ib & 0x7fff), ib)
    return (ia - ib).abs()


def test_layernorm_affine_vs_float64_and_group_indexing():
    g = torch.Generator().manual_seed(3)
    m, k, rpg = 37, 512, 10
    x = (torch.randn(m, k, generator=g) * 3 + 0.7).bfloat16()
    mul = 1 + 0.3 * torch.randn(4, k, generator=g)
    add = 0.2 * torch.randn(4, k, generator=g)
    y = O.layernorm_affine_bf16(x, mul, add, rpg, 1e-6)
    xd = x.double().numpy()
    mean = xd.mean(1, keepdims=True)
    var = ((xd - mean) ** 2).mean(1, keepdims=True)   # biased variance
    grp = np.arange(m) // rpg
    ref = (xd - mean) / np.sqrt(var + 1e-6) * mul.double().numpy()[grp] + add.double().numpy()[grp]
    ref_bf16 = torch.from_numpy(ref).float().bfloat16()
    ulps = _bf16_ulps(y, ref_bf16)
    assert int(ulps.max()) <= 1                      # only rounding-boundary cases may differ
    assert float((ulps > 0).float().mean()) < 2e-3
    # a wrong group index, a dropped term or an unbiased variance moves far more than that
    wrong = (xd - mean) / np.sqrt(xd.var(1, ddof=1, keepdims=True) + 1e-6) * mul.double().numpy()[grp] + add.double().numpy()[grp]
    assert float((_bf16_ulps(y, torch.from_numpy(wrong).float().bfloat16()) > 0).float().mean()) > 0.05


def test_layernorm_constant_row_and_missing_vectors():
    x = torch.full((3, 64), 2.5).bfloat16()
    add = torch.linspace(-1, 1, 64).reshape(1, 64)
    y = O.layernorm_affine_bf16(x, None, add, 3, 1e-6)
    assert torch.equal(y, add.bfloat16().expand(3, 64))         # (x - mean) is exactly zero
    y2 = O.layernorm_affine_bf16(torch.tensor([[1.0, -1.0] * 4]).bfloat16(), None, None, 1, 0.0)
    assert torch.equal(y2.float(), torch.tensor([[1.0, -1.0] * 4]))  # mean 0, variance 1


def test_gelu_tanh_every_bf16_input_vs_float64():
    bits = torch.arange(0, 1 << 16, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16)
    x = x[torch.isfinite(x.float())]
    y = O.gelu_tanh_bf16(x)
    xd = x.double().numpy()
    ref = 0.5 * xd * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (xd + 0.044715 * xd ** 3)))
    ref_bf16 = torch.from_numpy(ref).float().bfloat16()
    # for x < -5.3 the fp32 evaluation of 1 + tanh(u) is exactly 0 and torch returns -0.0 where the
    # true value is a negative number below 1e-7: counted as equal (absolute criterion), elsewhere
    # at most one bf16 step at rounding boundaries
    ulps = _bf16_ulps(y, ref_bf16)
    tiny = (y.double() - torch.from_numpy(ref)).abs() < 1e-6
    assert bool(((ulps <= 1) | tiny).all())
    assert float(((ulps > 0) & ~tiny).float().mean()) < 5e-3
    # a bf16 input is evaluated in fp32 and rounded once: the same as torch applied to the bf16 tensor
    assert torch.equal(y.view(torch.int16), torch.nn.functional.gelu(x, approximate="tanh").view(torch.int16))
    # known answers
    one = O.gelu_tanh_bf16(torch.tensor([0.0, 1.0, -1.0, 10.0, -10.0]).bfloat16()).float()
    assert one[0] == 0 and abs(float(one[1]) - 0.8412) < 4e-3 and abs(float(one[2]) + 0.1588) < 1e-3
    assert one[3] == 10.0 and one[4] == 0.0
    # the erf form is a different function: the tanh form must not silently be replaced by it
    mid = (x.float().abs() > 0.5) & (x.float().abs() < 4)
    erf = torch.nn.functional.gelu(x.float()).bfloat16()
    assert float((_bf16_ulps(y, erf)[mid] > 0).float().mean()) > 0.15
