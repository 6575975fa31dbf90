"""Pins for the torch-CPU oracle (oracle/daxq_oracle.py).

The reference holds no tests, golden vectors or fixtures for this path, so the
oracle is pinned by what the mathematics fixes: each torch-op restatement must
agree, exhaustively where the domain allows, with the hand-rounded bit-level C
closed form in oracle/daxq_oracle_c.c, with numpy brute force, and with known
answers.  A dropped rounding step, a reciprocal in place of a division, a wrong
tie rule or a transposed operand fails at least one test here.
"""
import numpy as np
import pytest
import torch

from oracle import daxq_oracle as O


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


ALL_POS_FINITE = np.arange(0, 0x7F80, dtype=np.uint16)  # +0 .. largest finite bf16


# ------------------------------------------------------------------ act scale
@pytest.mark.parametrize("qmax", [127.0, 448.0])
def test_act_scale_exhaustive_all_bf16_amax(closed_form, qmax):
    # a one-column "row" per amax value: the row abs-max is the value itself
    x = from_bits(ALL_POS_FINITE).view(-1, 1)
    got = O.act_scale(x, qmax).view(-1).numpy()
    want = closed_form.act_scale_vec(ALL_POS_FINITE, qmax)
    assert got.dtype == np.float32
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    # the scale is bf16-representable (low 16 bits clear) and floored at 2^-23
    assert not (got.view(np.uint32) & 0xFFFF).any()
    assert got.min() == np.float32(2.0 ** -23)
    # the bf16 rounding is live: an fp32 scale would differ for most amax values
    f32_scale = np.maximum((x.float().view(-1) / qmax).numpy(), np.float32(2.0 ** -23))
    assert (f32_scale != got).mean() > 0.4


def test_act_scale_uses_abs_and_row_max():
    x = torch.tensor([[1.0, -3.0, 2.0], [0.0, 0.0, 0.0], [-0.5, 0.25, 0.125]]).bfloat16()
    s = O.act_scale(x, 127.0).view(-1)
    assert s[0] == torch.tensor(3.0 / 127.0).bfloat16().float()
    assert s[1] == 2.0 ** -23  # zero row -> eps
    assert s[2] == torch.tensor(0.5 / 127.0).bfloat16().float()


# ------------------------------------------------------------------ int8 leaf
def reachable_scales(qmax):
    x = from_bits(ALL_POS_FINITE).view(-1, 1)
    return np.unique(O.act_scale(x, qmax).view(-1).numpy())


def test_quant_int8_closed_form_all_bf16_x_sampled_scales(closed_form):
    scales = reachable_scales(127.0)
    assert 15000 < scales.size < 20000
    rng = np.random.default_rng(0)
    pick = np.concatenate([scales[:4], scales[-4:], rng.choice(scales, 120, replace=False)])
    finite = np.concatenate([np.arange(0, 0x7F80), np.arange(0x8000, 0xFF80)]).astype(np.uint16)
    xt = from_bits(finite)
    for s in pick:
        # only x with |x| <= the largest amax that maps to this scale are reachable,
        # but the closed form holds for every finite x, so test them all
        got = O.quantize_to_int8(xt, torch.tensor([float(s)], dtype=torch.float32)).numpy()
        want = closed_form.quant_i8_vec(finite, float(s))
        np.testing.assert_array_equal(got, want)


def test_quant_int8_amax_maps_to_127_never_minus_128(closed_form):
    amax = ALL_POS_FINITE[ALL_POS_FINITE > 0]
    x = from_bits(amax).view(-1, 1)
    s = O.act_scale(x, 127.0)
    live = (s.view(-1) > 2.0 ** -23).numpy()
    q_pos = O.quantize_to_int8(x, s).view(-1).numpy()
    q_neg = O.quantize_to_int8(-x, s).view(-1).numpy()
    assert (q_pos[live] == 127).all() and (q_neg[live] == -127).all()
    assert q_neg.min() >= -127  # -128 is unreachable through the dynamic path


def test_quant_int8_round_half_even_and_reciprocal():
    s = torch.tensor([0.5], dtype=torch.float32)  # inv = 2 exactly (1-d: a 0-d scale would not promote bf16 to fp32)
    x = torch.tensor([0.25, 0.75, 1.25, -0.25, -0.75, 100.0, -100.0]).bfloat16()
    q = O.quantize_to_int8(x, s)
    assert q.tolist() == [0, 2, 2, 0, -2, 127, -128]
    # reciprocal-multiply differs from true division for some (x, fp32 scale) pairs, which the
    # weight path (un-rounded fp32 scales) can reach: the oracle must follow the reciprocal form
    g = torch.Generator().manual_seed(0)
    sc = (torch.rand(4000, 1, generator=g) * 0.01 + 1e-4)
    xs = from_bits(np.arange(0x3C00, 0x3F80, dtype=np.uint16)).view(1, -1)
    a = torch.clamp(torch.round(xs.float() * (1.0 / sc)), -128, 127)
    b = torch.clamp(torch.round(xs.float() / sc), -128, 127)
    assert (a != b).any()
    got = O.quantize_to_int8(xs.expand(4000, -1), sc)
    assert torch.equal(got, a.to(torch.int8))


# ------------------------------------------------------------------ fp8 leaf
def test_e4m3_decode_table_matches_torch(closed_form):
    table = closed_form.e4m3fn_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(table.view(np.uint32)[~np.isnan(table)], tt.view(np.uint32)[~np.isnan(tt)])
    assert np.isnan(table[[0x7F, 0xFF]]).all() and np.isnan(tt[[0x7F, 0xFF]]).all()
    assert table[0x7E] == 448.0 and table[0x01] == 2.0 ** -9 and table[0x08] == 2.0 ** -6


def test_e4m3_cast_known_answers(closed_form):
    v = np.array([448, 464, 17, 19, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -9, 0.0, -0.0, 18, 22, 26,
                  -448, 1.0, 0.0625 * 1.0625, 2.0 ** -6 - 2.0 ** -10], np.float32)
    want_f = np.array([448, 448, 16, 20, 0.0, 2.0 ** -9, 2.0 ** -9, 0.0, -0.0, 18, 22, 26,
                       -448, 1.0, 0.0625, 2.0 ** -6], np.float32)
    got_c = closed_form.e4m3fn_table()[closed_form.f32_to_e4m3fn(v)]
    got_t = torch.from_numpy(v).to(torch.float8_e4m3fn).float().numpy()
    np.testing.assert_array_equal(got_c, want_f)
    np.testing.assert_array_equal(got_t, want_f)
    assert np.isnan(torch.tensor([465.0]).to(torch.float8_e4m3fn).float().item())
    assert closed_form.f32_to_e4m3fn(np.array([465.0], np.float32))[0] == 0x7F


def test_e4m3_cast_dense_f32_sweep_torch_vs_closed_form(closed_form):
    # every f32 bit pattern with |v| <= 464 at stride 97 (coprime with 2^k), plus every
    # pattern within +-64 ulps of each tie point / representable value
    hi = np.float32(464.0).view(np.uint32)
    pats = np.arange(0, int(hi) + 1, 97, dtype=np.uint32)
    table = closed_form.e4m3fn_table()
    vals = np.unique(np.abs(table[~np.isnan(table)]))
    mids = (vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2
    anchors = np.concatenate([vals, mids.astype(np.float32), [np.float32(2.0 ** -10)]]).astype(np.float32)
    near = (anchors.view(np.uint32)[:, None].astype(np.int64) + np.arange(-64, 65)[None, :]).reshape(-1)
    near = near[(near >= 0) & (near <= int(hi))].astype(np.uint32)
    pats = np.unique(np.concatenate([pats, near]))
    for sign in (0, 0x80000000):
        v = (pats | np.uint32(sign)).view(np.float32)
        got_t = torch.from_numpy(v.copy()).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        got_c = closed_form.f32_to_e4m3fn(v)
        np.testing.assert_array_equal(got_t, got_c)


def test_quant_fp8_closed_form_all_bf16_x_sampled_scales(closed_form):
    scales = reachable_scales(448.0)
    rng = np.random.default_rng(1)
    pick = np.concatenate([scales[:4], scales[-4:], rng.choice(scales, 120, replace=False)])
    finite = np.concatenate([np.arange(0, 0x7F80), np.arange(0x8000, 0xFF80)]).astype(np.uint16)
    xt = from_bits(finite)
    for s in pick:
        got = O.quantize_to_fp8(xt, torch.tensor([float(s)], dtype=torch.float32)).view(torch.uint8).numpy()
        want = closed_form.quant_e4m3_vec(finite, float(s))
        np.testing.assert_array_equal(got, want)


def test_quant_fp8_clamp_is_live_and_saturates_to_448():
    amax = ALL_POS_FINITE[ALL_POS_FINITE > 0]
    x = from_bits(amax).view(-1, 1)
    s = O.act_scale(x, 448.0)
    ratio = (x.float() / s).view(-1)
    live = (s.view(-1) > 2.0 ** -23)
    assert (ratio[live] > 448).any() and ratio[live].max() <= 464  # clamp needed, never NaN
    q = O.quantize_to_fp8(x, s).float().view(-1)
    assert (q[live] == 448).all()
    # true division, not reciprocal multiply
    xs = torch.tensor([3.0]).bfloat16()
    sc = torch.tensor([3.0], dtype=torch.float32)
    assert O.quantize_to_fp8(xs, sc).float().item() == 1.0


# ------------------------------------------------------------------ e5m2 (the FP8 qconfig's default activation dtype)
def test_e5m2_cast_torch_vs_closed_form(closed_form):
    table = closed_form.e5m2_table()
    tt = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).float().numpy()
    ok = ~np.isnan(table)
    np.testing.assert_array_equal(table[ok].view(np.uint32), tt[ok].view(np.uint32))
    assert table[0x7B] == 57344.0 and table[0x01] == 2.0 ** -16 and np.isinf(table[0x7C])
    v = np.array([57344, 61439.9, 61440, 3.0, 3.5, 4.5, 2.0 ** -17, 1.5 * 2.0 ** -17, 2.0 ** -16, -57344, 1.125, 1.375],
                 np.float32)
    want = np.array([57344, 57344, np.inf, 3.0, 3.5, 4.0, 0.0, 2.0 ** -16, 2.0 ** -16, -57344, 1.0, 1.5], np.float32)
    np.testing.assert_array_equal(table[closed_form.f32_to_e5m2(v)], want)
    np.testing.assert_array_equal(torch.from_numpy(v).to(torch.float8_e5m2).float().numpy(), want)
    hi = np.float32(61440.0).view(np.uint32)
    pats = np.arange(0, int(hi) + 2048, 53, dtype=np.uint32)
    vals = np.unique(np.abs(table[np.isfinite(table)]))
    mids = ((vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2).astype(np.float32)
    near = (np.concatenate([vals, mids]).view(np.uint32)[:, None].astype(np.int64) + np.arange(-64, 65)[None, :]).reshape(-1)
    near = near[(near >= 0) & (near <= int(hi) + 2048)].astype(np.uint32)
    pats = np.unique(np.concatenate([pats, near]))
    for sign in (0, 0x80000000):
        f = (pats | np.uint32(sign)).view(np.float32)
        got_t = torch.from_numpy(f.copy()).to(torch.float8_e5m2).view(torch.uint8).numpy()
        np.testing.assert_array_equal(got_t, closed_form.f32_to_e5m2(f))


def test_quant_e5m2_closed_form_all_bf16_x_sampled_scales(closed_form):
    scales = reachable_scales(57344.0)
    rng = np.random.default_rng(2)
    pick = np.concatenate([scales[:4], scales[-4:], rng.choice(scales, 100, replace=False)])
    finite = np.concatenate([np.arange(0, 0x7F80), np.arange(0x8000, 0xFF80)]).astype(np.uint16)
    xt = from_bits(finite)
    for s in pick:
        got = O.quantize_to_fp8(xt, torch.tensor([float(s)], dtype=torch.float32), torch.float8_e5m2)
        np.testing.assert_array_equal(got.view(torch.uint8).numpy(), closed_form.quant_e5m2_vec(finite, float(s)))
    # +-amax lands on +-57344 (never inf): the clamp is what keeps it finite
    amax = ALL_POS_FINITE[ALL_POS_FINITE > 0]
    x = from_bits(amax).view(-1, 1)
    s = O.act_scale(x, 57344.0)
    live = (s.view(-1) > 2.0 ** -23)
    q = O.quantize_to_fp8(x, s, torch.float8_e5m2).float().view(-1)
    assert (q[live] == 57344).all() and ((x.float() / s).view(-1)[live] > 57344).any()


def test_act_quant_e5m2_rows_vs_closed_form(closed_form):
    x, _, _ = O.make_inputs(48, 320, 8, seed=13)
    x[3] = 0
    q, s = O.act_quant_e5m2(x)
    qc, sc = closed_form.act_quant_e5m2(bf16_bits(x))
    np.testing.assert_array_equal(q.view(torch.uint8).numpy(), qc)
    np.testing.assert_array_equal(s.view(-1).numpy(), sc)
    assert q.dtype == torch.float8_e5m2


# ------------------------------------------------------------------ whole rows
def test_act_quant_rows_vs_closed_form(closed_form):
    x, _, _ = O.make_inputs(64, 384, 8, seed=3)
    x[5] = 0  # zero row
    x[6, :] = 0
    x[6, 17] = -1e-30  # tiny row below the eps floor
    q, s = O.act_quant_int8(x)
    qc, sc = closed_form.act_quant_i8(bf16_bits(x))
    np.testing.assert_array_equal(q.numpy(), qc)
    np.testing.assert_array_equal(s.view(-1).numpy(), sc)
    assert (q[5] == 0).all() and s[5] == 2.0 ** -23
    q8, s8 = O.act_quant_e4m3(x)
    qc8, sc8 = closed_form.act_quant_e4m3(bf16_bits(x))
    np.testing.assert_array_equal(q8.view(torch.uint8).numpy(), qc8)
    np.testing.assert_array_equal(s8.view(-1).numpy(), sc8)


def test_act_quant_keeps_leading_dims_flat():
    x, _, _ = O.make_inputs(24, 64, 8, seed=4)
    q3, s3 = O.act_quant_int8(x.view(2, 12, 64))
    q2, s2 = O.act_quant_int8(x)
    assert torch.equal(q3, q2) and torch.equal(s3, s2) and s2.shape == (24, 1)


# ------------------------------------------------------------------ weights
@pytest.mark.parametrize("qmax", [127.0, 448.0])
def test_weight_scale_vs_closed_form_and_no_bf16_rounding(closed_form, qmax):
    _, w, _ = O.make_inputs(4, 256, 96, seed=5)
    w[3] = 0
    w[4, 0] = -2.0  # negative extreme decides the scale
    s = O.weight_scale(w, qmax).numpy()
    np.testing.assert_array_equal(s, closed_form.weight_scale(bf16_bits(w), qmax))
    assert s[3] == np.float32(2.0 ** -23)
    assert s[4] == np.float32(2.0) / np.float32(qmax)
    assert (s.view(np.uint32) & 0xFFFF).any()  # fp32 scale, not bf16-rounded


def test_weight_quant_int8_rows(closed_form):
    _, w, _ = O.make_inputs(4, 128, 32, seed=6)
    q, s = O.weight_quant_int8(w)
    assert q.shape == (32, 128) and s.shape == (1, 32) and s.dtype == torch.float32
    wb = bf16_bits(w)
    for r in range(32):
        np.testing.assert_array_equal(q[r].numpy(), closed_form.quant_i8_vec(wb[r], float(s[0, r])))
    q8, s8 = O.weight_quant_e4m3(w)
    for r in range(32):
        np.testing.assert_array_equal(q8[r].view(torch.uint8).numpy(),
                                      closed_form.quant_e4m3_vec(wb[r], float(s8[0, r])))


def test_dequant_weight_property():
    _, w, _ = O.make_inputs(4, 64, 16, seed=7)
    q, s = O.weight_quant_int8(w)
    d = O.dequant_weight(q, s)
    assert d.dtype == torch.bfloat16 and d.shape == w.shape
    assert torch.equal(d, q.bfloat16() * s.view(-1, 1).bfloat16())
    assert (d.float() - w.float()).abs().max() <= s.max() * 0.51 + 1e-3


# ------------------------------------------------------------------ int GEMM
@pytest.mark.parametrize("m,n,k", [(1, 8, 16), (17, 24, 64), (33, 40, 200)])
def test_int_mm_vs_bruteforce(closed_form, m, n, k):
    rng = np.random.default_rng(m * 1000 + k)
    a = rng.integers(-128, 128, (m, k), dtype=np.int8)
    b = rng.integers(-128, 128, (n, k), dtype=np.int8)
    got = O.int_mm(torch.from_numpy(a), torch.from_numpy(b)).numpy()
    want64 = a.astype(np.int64) @ b.astype(np.int64).T
    np.testing.assert_array_equal(got.astype(np.int64), want64)
    np.testing.assert_array_equal(closed_form.gemm_i8(a, b), got)


def test_int_mm_adversarial_extremes_no_overflow():
    k = 13824
    a = np.full((32, k), -128, np.int8)
    b = np.full((8, k), -128, np.int8)
    b[1] = 127
    got = O.int_mm(torch.from_numpy(a), torch.from_numpy(b)).numpy()
    assert (got[:, 0] == 128 * 128 * k).all() and (got[:, 1] == -128 * 127 * k).all()
    assert 128 * 128 * k < 2 ** 31


def test_int_mm_is_x_times_w_transposed():
    a = torch.zeros(20, 32, dtype=torch.int8)
    b = torch.zeros(24, 32, dtype=torch.int8)
    a[3, 5] = 2
    b[7, 5] = 3
    out = O.int_mm(a, b)
    assert out.shape == (20, 24) and out[3, 7] == 6 and out.abs().sum() == 6


# ------------------------------------------------------------------ epilogue
def test_epilogue_int8_closed_form_double_rounding(closed_form):
    rng = np.random.default_rng(9)
    m, n = 48, 64
    acc = rng.integers(-2 ** 28, 2 ** 28, (m, n), dtype=np.int32)  # > 2^24: the convert rounds
    acc[0, :8] = [16777217, -16777217, 16777219, 2 ** 28 - 1, 0, 1, -1, 33554435]
    sx = from_bits(rng.integers(0x3800, 0x3E00, m).astype(np.uint16)).float()
    sw = torch.from_numpy(rng.random(n, dtype=np.float32) * 1e-3 + 1e-5)
    bias = (torch.randn(n, generator=torch.Generator().manual_seed(9)) * 0.01).bfloat16()
    got = O.epilogue_int8(torch.from_numpy(acc), sx.view(-1, 1), sw.view(1, -1), bias)
    want = closed_form.epilogue_i8(acc, sx.numpy(), sw.numpy(), bf16_bits(bias))
    assert got.dtype == torch.bfloat16
    np.testing.assert_array_equal(bf16_bits(got), want)
    got_nb = O.epilogue_int8(torch.from_numpy(acc), sx.view(-1, 1), sw.view(1, -1), None)
    np.testing.assert_array_equal(bf16_bits(got_nb), closed_form.epilogue_i8(acc, sx.numpy(), sw.numpy(), None))
    # the bias add is a second bf16 rounding, not fused into the first
    fused = (torch.from_numpy(acc).float() * sx.view(-1, 1) * sw.view(1, -1) + bias.float()).bfloat16()
    assert (bf16_bits(fused) != bf16_bits(got)).any()


def test_linear_int8_end_to_end_small(closed_form):
    x, w, b = O.make_inputs(40, 256, 48, seed=11)
    qw, sw = O.weight_quant_int8(w)
    r = O.linear_int8(x, qw, sw, b, row_chunk=16)
    qc, sc = closed_form.act_quant_i8(bf16_bits(x))
    acc = closed_form.gemm_i8(qc, qw.numpy())
    np.testing.assert_array_equal(r["acc"].numpy(), acc)
    np.testing.assert_array_equal(bf16_bits(r["out"]), closed_form.epilogue_i8(acc, sc, sw.numpy(), bf16_bits(b)))
    # close to the float linear it replaces
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    rel = (r["out"].float() - ref).norm() / ref.norm()
    assert rel < 5e-2  # quantisation error against the float layer, not a parity bound


# ------------------------------------------------------------------ fp8 linear
def test_linear_e4m3_matches_float_and_per_tensor_scaled_mm():
    x, w, b = O.make_inputs(64, 256, 48, seed=12)
    qw, sw = O.weight_quant_e4m3(w)
    r = O.linear_e4m3(x, qw, sw, b)
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    rel = (r["out"].float() - ref).norm() / ref.norm()
    assert rel < 1e-1  # e4m3 has 3 mantissa bits
    # library special case: per-tensor scales reduce to torch._scaled_mm on CPU
    xq = r["xq"][:32].contiguous()
    one = torch.tensor(0.5), torch.tensor(0.25)
    try:
        lib = torch._scaled_mm(xq, qw.t(), scale_a=one[0], scale_b=one[1], out_dtype=torch.bfloat16)
    except (RuntimeError, NotImplementedError) as e:  # pragma: no cover
        pytest.skip(f"torch._scaled_mm not available on this CPU build: {e}")
    emu = ((xq.float() @ qw.float().t()) * 0.5 * 0.25).bfloat16()
    assert ((lib.float() - emu.float()).norm() / emu.float().norm()) < 1e-2


def test_make_inputs_is_seeded_and_has_outliers():
    x1, w1, b1 = O.make_inputs(256, 1536, 16, seed=0)
    x2, _, _ = O.make_inputs(256, 1536, 16, seed=0)
    assert torch.equal(x1, x2) and x1.dtype == torch.bfloat16
    col_std = x1.float().std(0)
    assert (col_std > 10).sum() == 15  # round(0.01 * 1536) outlier channels, x20
    assert abs(w1.float().std().item() - 0.02) < 2e-3 and abs(b1.float().std().item() - 0.01) < 5e-3


def test_per_tensor_scales_reduce_to_the_per_row_functions():
    """A per-tensor block is the per-row rule applied to the tensor flattened into one row."""
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(37, 96, generator=g) * 5).bfloat16()
    for qmax in (O.INT8_QMAX, O.E4M3_QMAX, O.E5M2_QMAX):
        assert torch.equal(O.act_scale_per_tensor(x, qmax), O.act_scale(x.reshape(1, -1), qmax).reshape(1))
        assert torch.equal(O.weight_scale_per_tensor(x, qmax), O.weight_scale(x.reshape(1, -1), qmax).reshape(1))
    z = torch.zeros(4, 8).bfloat16()
    assert float(O.act_scale_per_tensor(z, 127)) == 2.0 ** -23 and float(O.weight_scale_per_tensor(z, 127)) == 2.0 ** -23
    # the four INT8 scheme pairs agree with the per-token / per-channel chain when every row / channel has the same amax
    x2 = torch.tensor([[1.0, -2.0, 4.0, 0.5]] * 3).bfloat16()
    w2 = torch.tensor([[0.5, -1.0, 0.25, 1.0]] * 5).bfloat16()
    b = torch.zeros(5).bfloat16()
    base = O.linear_int8_schemes(x2, w2, b, False, False)["out"]
    for ap, wp in ((True, False), (False, True), (True, True)):
        assert torch.equal(O.linear_int8_schemes(x2, w2, b, ap, wp)["out"], base)


def test_static_linear_fp8_matches_the_float_layer():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(64, 128, generator=g).bfloat16()
    w = (torch.randn(32, 128, generator=g) * 0.05).bfloat16()
    b = (torch.randn(32, generator=g) * 0.01).bfloat16()
    si = O.weight_scale_per_tensor(x, O.E4M3_QMAX)                 # what a MinMaxObserver calibrated on x gives
    sw = O.weight_scale_per_tensor(w, O.E4M3_QMAX)
    qw = O.quantize_to_fp8(w, sw)
    out = O.static_linear_fp8(x, si, qw, sw, b)["out"]
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    assert float((out.float() - ref).norm() / ref.norm()) < 6e-2    # fp8 (3 mantissa bits) quantisation error
    # per-tensor special case of the library routine on CPU
    lib = torch._scaled_mm(O.quantize_to_fp8(x, si), qw.t(), scale_a=si.reshape(()), scale_b=sw.reshape(()), bias=b,
                           out_dtype=torch.bfloat16)
    assert float((out.float() - lib.float()).norm() / lib.float().norm()) < 4e-3

