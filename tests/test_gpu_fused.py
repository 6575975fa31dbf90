"""GPU tests of the fused producer + quantiser kernels, through torch.ops.daxq -> C ABI.

Two-part check.  The producer (LayerNorm multiply-add, GELU-tanh) is floating point: its bf16 result y
must agree with the oracle to one bf16 step, and only at rounding boundaries (stated fractions below).
The quantiser behind it is integer work: the scales and quantised bytes the kernel returns must equal,
bit for bit, the oracle's quantiser applied to the kernel's own y.
"""
import pytest
import torch

from oracle import daxq_oracle as O
from tests.util import FINITE_BF16, bf16_ulps, from_bits, rel_l2

pytestmark = pytest.mark.gpu

QUANT = {"i8": O.act_quant_int8, "e4m3": O.act_quant_e4m3, "e5m2": O.act_quant_e5m2}


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import dax_amd.ops as ops

    return ops


def dev(t):
    return None if t is None else t.to("cuda")


def _check_quant_of_own_y(fmt, y_gpu, q_gpu, s_gpu, k):
    q_ref, s_ref = QUANT[fmt](y_gpu.cpu())
    assert torch.equal(s_gpu.cpu(), s_ref.view(-1))
    q_ref = q_ref if fmt == "i8" else q_ref.view(torch.uint8)
    assert torch.equal(q_gpu[:, :k].cpu(), q_ref)
    assert int(q_gpu[:, k:].cpu().to(torch.int32).abs().sum()) == 0       # K padding is zero


def _check_y(y_gpu, y_ref, max_frac):
    ulps = bf16_ulps(y_gpu, y_ref)
    tiny = (y_gpu.cpu().double() - y_ref.double()).abs() < 1e-6
    assert bool(((ulps <= 1) | tiny).all()), int(ulps.max())
    frac = float(((ulps > 0) & ~tiny).float().mean())
    assert frac < max_frac, frac


@pytest.mark.parametrize("fmt", ["i8", "e4m3", "e5m2"])
def test_gelu_tanh_every_bf16_input(ops, fmt):
    x = from_bits(FINITE_BF16)
    pad = (-x.numel()) % 1024
    x = torch.cat([x, x[:pad]]).reshape(-1, 1024)
    q, s, y = getattr(ops, "gelu_tanh_act_quant_" + fmt)(dev(x), True)
    _check_y(y, O.gelu_tanh_bf16(x), 1e-2)
    _check_quant_of_own_y(fmt, y, q, s, 1024)


@pytest.mark.parametrize("fmt", ["i8", "e4m3", "e5m2"])
@pytest.mark.parametrize("m,k", [(130, 13824), (257, 8960), (33, 1536), (1, 8), (5, 200), (41, 6144), (9, 8192), (22, 12288)])
def test_gelu_tanh_shapes_and_quant_only_form(ops, fmt, m, k):
    """The form that writes only the quantised bytes takes a kernel of its own for rows of 12, 16, 24 or 27 whole
    512-element columns (K = 13824 and the last three shapes); its bytes and scales must equal those of the general kernel,
    which writes y as well."""
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) * 1.5).bfloat16()
    fn = getattr(ops, "gelu_tanh_act_quant_" + fmt)
    q, s, y = fn(dev(x), True)
    _check_y(y, O.gelu_tanh_bf16(x), 1e-2)
    _check_quant_of_own_y(fmt, y, q, s, k)
    q2, s2, y2 = fn(dev(x), False)                                        # without writing y
    assert y2.shape[0] == 0 and torch.equal(q2, q) and torch.equal(s2, s)


@pytest.mark.parametrize("fmt", ["i8", "e4m3", "e5m2"])
@pytest.mark.parametrize("m,k,rpg,vecs", [(300, 1536, 300, "both"), (1001, 5120, 333, "both"), (64, 5120, 64, "none"),
                                          (9, 256, 2, "mul"), (1, 8, 1, "add"), (70, 8192, 35, "both"),
                                          (9000, 1536, 3000, "both"), (5000, 5120, 2500, "both"), (130, 3072, 4, "mul"),
                                          (40, 8192, 8, "both"), (36, 2048, 12, "add"), (20, 4096, 20, "both"), (24, 6144, 24, "mul")])
def test_layernorm_multiply_add(ops, fmt, m, k, rpg, vecs):
    """Rows of whole 512-element columns in groups of a multiple of four rows take a kernel of their own when only the
    quantised bytes are asked for (from the seventh shape on: every column count it is built for, resident workgroups
    that make several passes, a group change at every pass); its bytes and scales must equal those of the general kernel, which writes y as well."""
    g = torch.Generator().manual_seed(m * 7 + k)
    x = (torch.randn(m, k, generator=g) * 2 + 0.3).bfloat16()
    x[:, :: max(1, k // 7)] *= 12                                         # outlier channels, as in the DiT
    groups = -(-m // rpg)
    mul = (1 + 0.2 * torch.randn(groups, k, generator=g)) if vecs in ("both", "mul") else None
    add = (0.1 * torch.randn(groups, k, generator=g)) if vecs in ("both", "add") else None
    fn = getattr(ops, "layernorm_act_quant_" + fmt)
    q, s, y = fn(dev(x), dev(mul), dev(add), rpg, 1e-6, True)
    _check_y(y, O.layernorm_affine_bf16(x, mul, add, rpg, 1e-6), 5e-3)
    _check_quant_of_own_y(fmt, y, q, s, k)
    q2, s2, _ = fn(dev(x), dev(mul), dev(add), rpg, 1e-6, False)
    assert torch.equal(q2, q) and torch.equal(s2, s)


@pytest.mark.parametrize("fmt", ["i8", "e4m3"])
def test_layernorm_rows_with_an_offset(ops, fmt):
    """The variance comes from sum(x^2) / K - mean^2 while the mean is small against the spread and from the second
    pass over the row otherwise: rows whose offset runs from none to a thousand times the spread (both sides of the
    switch at mean^2 = 7 var), a row that is constant but for one element, tiny and huge magnitudes."""
    g = torch.Generator().manual_seed(11)
    k = 5120
    offsets = [0.0, 0.5, 1.0, 2.0, 2.5, 2.6, 2.7, 3.0, 4.0, 10.0, 100.0, 1000.0, -2.6, -50.0]
    rows = [torch.randn(k, generator=g) + o for o in offsets]
    rows += [torch.randn(k, generator=g) * 1e-3 + 1.0, torch.randn(k, generator=g) * 300 + 5e4, torch.randn(k, generator=g) * 1e-20]
    spike = torch.full((k,), 7.0)
    spike[123] = 9.0
    rows.append(spike)
    x = torch.stack(rows).bfloat16()
    mul = 1 + 0.2 * torch.randn(1, k, generator=g)
    add = 0.1 * torch.randn(1, k, generator=g)
    fn = getattr(ops, "layernorm_act_quant_" + fmt)
    q, s, y = fn(dev(x), dev(mul), dev(add), x.shape[0], 1e-6, True)
    # Against the exact result (float64): torch's CPU kernel, which the oracle calls, evaluates x * rstd - mean * rstd
    # and loses digits to that cancellation once the offset is 50 times the spread; (x - mean) * rstd, which the
    # kernel and torch's GPU kernel evaluate, does not.
    xd = x.double()
    mean = xd.mean(1, keepdim=True)
    exact = ((xd - mean) / (xd.var(1, unbiased=False, keepdim=True) + 1e-6).sqrt() * mul.double() + add.double()).float().bfloat16()
    ref = O.layernorm_affine_bf16(x, mul, add, x.shape[0], 1e-6)
    rstd = (xd.var(1, unbiased=False, keepdim=True) + 1e-6).rsqrt()
    for r in range(x.shape[0]):          # row by row: the bound on the share of one-step differences holds for every row
        # an fp32 mean resolves 6e-8 of itself, so x - mean carries that much absolute error, times rstd and mul: it
        # shows only where the output lies next to zero (the multiply-add cancels), where bf16 steps are tiny
        tol = max(1e-6, 2.4e-7 * abs(float(mean[r])) * float(rstd[r]))
        diff = (y[r].cpu().double() - exact[r].double()).abs()
        ulps = bf16_ulps(y[r:r + 1], exact[r:r + 1]).view(-1)
        assert bool(((ulps <= 1) | (diff < tol)).all()), (r, int(ulps.max()), float(diff.max()), tol)
        # (rows 11, 14 and 17 hold two to five distinct bf16 values, so their outputs sit in as many narrow clusters and a
        # cluster next to a rounding boundary is several per cent of the row at once)
        assert float(((ulps > 0) & (diff >= tol)).float().mean()) < (5e-2 if r in (11, 14, 17) else 1e-2), r
        if r < 10:                       # offsets up to ten times the spread: the oracle agrees as well
            _check_y(y[r:r + 1], ref[r:r + 1], 1e-2)
    _check_quant_of_own_y(fmt, y, q, s, k)


def test_layernorm_constant_rows_and_strided_input(ops):
    x = torch.full((8, 512), -3.0).bfloat16()
    add = torch.linspace(-2, 2, 512).reshape(1, 512)
    q, s, y = ops.layernorm_act_quant_i8(dev(x), None, dev(add), 8, 1e-6, True)
    assert torch.equal(y.cpu(), add.bfloat16().expand(8, 512))
    big = torch.randn(16, 1024).bfloat16()
    xs = dev(big)[:, :512]                                                # row stride 1024
    q, s, y = ops.layernorm_act_quant_i8(xs, None, None, 16, 1e-6, True)
    _check_y(y, O.layernorm_affine_bf16(big[:, :512].contiguous(), None, None, 16, 1e-6), 5e-3)


def test_fused_inputs_of_a_linear_end_to_end(ops):
    """norm -> modulate -> quantised linear and gelu -> quantised linear against the unfused oracle chain."""
    m, k, n = 512, 1536, 1024
    x, w, b = O.make_inputs(m, k, n, seed=11)
    g = torch.Generator().manual_seed(5)
    mul, add = 1 + 0.1 * torch.randn(1, k, generator=g), 0.05 * torch.randn(1, k, generator=g)
    qw, sw = O.weight_quant_int8(w)
    for name, y_ref, call in [
        ("layernorm", O.layernorm_affine_bf16(x, mul, add, m, 1e-6),
         lambda: ops.layernorm_act_quant_i8(dev(x), dev(mul), dev(add), m, 1e-6)),
        ("gelu", O.gelu_tanh_bf16(x), lambda: ops.gelu_tanh_act_quant_i8(dev(x))),
    ]:
        ref = O.linear_int8(y_ref, qw, sw, b)["out"]
        xq, sx, _ = call()
        out = ops.linear_i8(xq, sx, dev(qw), dev(sw.view(-1)), dev(b))
        assert rel_l2(out, ref) < 5e-3, name      # a flipped rounding of y moves one int8 step in one row


def test_fused_errors_are_loud(ops):
    x = torch.randn(4, 16384).bfloat16()
    with pytest.raises(RuntimeError):
        ops.gelu_tanh_act_quant_i8(dev(x))        # row too long for the register-resident kernel
    with pytest.raises(RuntimeError):
        ops.gelu_tanh_act_quant_i8(torch.randn(4, 64).bfloat16())   # CPU tensor
    with pytest.raises(ValueError):
        ops.layernorm_act_quant_i8(dev(torch.randn(4, 64).bfloat16()), dev(torch.ones(3, 64)), None, 4, 1e-6)
