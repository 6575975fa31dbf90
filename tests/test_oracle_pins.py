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
def decode_fp8(bits: np.ndarray, ebits: int) -> np.ndarray:
    """OCP e4m3fn (ebits 4) / e5m2 (ebits 5) bytes -> float64, from the bit layout alone: sign, biased
    exponent, mantissa; exponent 0 is subnormal.  e4m3fn has no infinities (S.1111.111 is NaN), e5m2 is IEEE-like."""
    b = bits.astype(np.int64)
    mbits = 7 - ebits
    bias = (1 << (ebits - 1)) - 1
    sign = np.where(b & 0x80, -1.0, 1.0)
    e = (b >> mbits) & ((1 << ebits) - 1)
    m = (b & ((1 << mbits) - 1)).astype(np.float64)
    val = np.where(e == 0, m * 2.0 ** (1 - bias - mbits), (1.0 + m * 2.0 ** -mbits) * 2.0 ** (e.astype(np.float64) - bias))
    if ebits == 4:
        val = np.where((b & 0x7F) == 0x7F, np.nan, val)
    else:
        val = np.where(e == 31, np.where(m == 0, np.inf, np.nan), val)
    return sign * val


def f64_to_bf16_bits_rne(y: np.ndarray) -> np.ndarray:
    """float64 -> bf16 bit pattern with ONE round-to-nearest-even (no intermediate float32 rounding):
    the two neighbouring bf16 values are built by truncating the float32 that lies at or below |y|."""
    y = np.asarray(y, np.float64)
    a = np.abs(y)
    f = a.astype(np.float32)
    f = np.where(f.astype(np.float64) > a, np.nextafter(f, np.float32(0)), f).astype(np.float32)  # f <= |y|
    lo = (f.view(np.uint32) >> 16).astype(np.uint32)  # bf16 at or below |y|
    lo_v = (lo << 16).astype(np.uint32).view(np.float32).astype(np.float64)
    hi_v = ((lo + 1) << 16).astype(np.uint32).view(np.float32).astype(np.float64)
    up = (a - lo_v > hi_v - a) | ((a - lo_v == hi_v - a) & ((lo & 1) == 1))
    mag = (lo + up.astype(np.uint32)).astype(np.uint16)
    return np.where(np.signbit(y), mag | 0x8000, mag).astype(np.uint16)


def ulps_apart(a_bits: np.ndarray, b_bits: np.ndarray) -> np.ndarray:
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a_bits) - key(b_bits))


def scaled_mm_exact(xq_bits, x_ebits, wq_bits, w_ebits, sa, sb, bias_bits):
    """bf16( sum_k dec(xq) dec(wq) * sa * sb + bias ) with every step in float64 and one final rounding."""
    acc = decode_fp8(xq_bits, x_ebits) @ decode_fp8(wq_bits, w_ebits).T
    y = acc * sa.astype(np.float64).reshape(-1, 1) * sb.astype(np.float64).reshape(1, -1)
    if bias_bits is not None:
        y = y + (bias_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64).reshape(1, -1)
    return f64_to_bf16_bits_rne(y)


def test_decode_and_rounding_helpers(closed_form):
    allb = np.arange(256, dtype=np.uint8)
    for ebits, table in ((4, closed_form.e4m3fn_table()), (5, closed_form.e5m2_table())):
        d = decode_fp8(allb, ebits)
        ok = ~np.isnan(table)
        np.testing.assert_array_equal(d[ok], table[ok].astype(np.float64))
        assert np.isnan(d[~ok]).all()
    # one rounding: a value just above a bf16 tie that float32 would first round onto the tie
    tie = np.float64(1.0) + 2.0 ** -8  # midway between bf16 1.0 and 1.0078125
    assert f64_to_bf16_bits_rne(np.array([tie]))[0] == 0x3F80  # tie -> even
    assert f64_to_bf16_bits_rne(np.array([tie + 2.0 ** -40]))[0] == 0x3F81  # float32 would see the tie
    assert f64_to_bf16_bits_rne(np.array([-tie - 2.0 ** -40]))[0] == 0xBF81
    v = np.random.default_rng(0).standard_normal(4096).astype(np.float32)
    np.testing.assert_array_equal(f64_to_bf16_bits_rne(v.astype(np.float64)), bf16_bits(torch.from_numpy(v).bfloat16()))


def _fp8_case(seed, m=96, k=384, n=80):
    """Rows / channels with scales spread over two decades and a bias as large as the outputs, so that a dropped
    bias, a dropped scale, a transposed scale or a second rounding each move many outputs."""
    x, w, _ = O.make_inputs(m, k, n, seed=seed)
    g = torch.Generator().manual_seed(seed + 100)
    x = (x.float() * torch.logspace(-1, 1, m).view(-1, 1)).bfloat16()
    w = (w.float() * torch.logspace(-1, 1, n).view(-1, 1)).bfloat16()
    b = (torch.randn(n, generator=g) * torch.nn.functional.linear(x.float(), w.float()).std()).bfloat16()
    return x, w, b


@pytest.mark.parametrize("act_dtype,w_dtype", [(torch.float8_e4m3fn, torch.float8_e4m3fn), (torch.float8_e5m2, torch.float8_e4m3fn),
                                               (torch.float8_e4m3fn, torch.float8_e5m2), (torch.float8_e5m2, torch.float8_e5m2)])
def test_linear_fp8_vs_float64_closed_form(act_dtype, w_dtype):
    """The FP8 forward against an evaluation from the decoded bytes in float64 with a single rounding: the fp32
    restatement may land on the other side of a bf16 rounding boundary (fp32 accumulation error ~1e-6 relative
    against the bf16 half-step 2e-3), never further."""
    x, w, b = _fp8_case(21)
    qw, sw = O.weight_quant_fp8(w, w_dtype)
    r = O.linear_fp8(x, qw, sw, b, act_dtype=act_dtype)
    eb = lambda dt: 4 if dt == torch.float8_e4m3fn else 5
    want = scaled_mm_exact(r["xq"].view(torch.uint8).numpy(), eb(act_dtype), qw.view(torch.uint8).numpy(), eb(w_dtype),
                           r["sx"].numpy(), sw.numpy(), bf16_bits(b))
    got = bf16_bits(r["out"])
    d = ulps_apart(got, want)
    assert d.max() <= 1 and (d != 0).mean() < 0.01, (d.max(), (d != 0).mean())
    # what the check is sensitive to: each of these restatement mistakes fails it
    acc = decode_fp8(r["xq"].view(torch.uint8).numpy(), eb(act_dtype)) @ decode_fp8(qw.view(torch.uint8).numpy(), eb(w_dtype)).T
    y = acc * r["sx"].numpy().astype(np.float64) * sw.numpy().astype(np.float64)
    bias64 = b.float().numpy().astype(np.float64)
    no_bias = f64_to_bf16_bits_rne(y)
    twice = f64_to_bf16_bits_rne((f64_to_bf16_bits_rne(y).astype(np.uint32) << 16).view(np.float32).astype(np.float64) + bias64)
    other = scaled_mm_exact(r["xq"].view(torch.uint8).numpy(), 9 - eb(act_dtype), qw.view(torch.uint8).numpy(), eb(w_dtype),
                            r["sx"].numpy(), sw.numpy(), bf16_bits(b))
    for name, wrong in (("no bias", no_bias), ("rounded twice", twice), ("other fp8 decoding", other)):
        dw = ulps_apart(got, wrong)
        assert dw.max() > 1 or (dw != 0).mean() >= 0.01, name
    # and it sits where a quantised layer should: close to the float layer it replaces
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    assert float((r["out"].float() - ref).norm() / ref.norm()) < (0.2 if torch.float8_e5m2 in (act_dtype, w_dtype) else 0.1)


def test_linear_fp8_per_tensor_is_the_library_scaled_mm():
    """Uniform scales reduce the forward to torch._scaled_mm with per-tensor scales, which the CPU build
    implements: the oracle function itself is called, with rows of equal abs-max and one weight scale."""
    x, w, b = _fp8_case(22, m=64, k=256, n=48)
    x[:, 0] = x.abs().max()  # every row has the same abs-max -> one activation scale
    for act_dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        sw1 = O.weight_scale_per_tensor(w, O.E4M3_QMAX)
        qw = O.quantize_to_fp8(w, sw1)
        for per_tensor in (False, True):
            r = O.linear_fp8(x, qw, sw1.expand(1, w.shape[0]) if not per_tensor else sw1, b, act_dtype=act_dtype,
                             per_tensor=per_tensor)
            sx = r["sx"].reshape(-1)
            assert (sx == sx[0]).all()
            try:
                lib = torch._scaled_mm(r["xq"], qw.t(), scale_a=sx[0].reshape(()), scale_b=sw1.reshape(()), bias=b,
                                       out_dtype=torch.bfloat16)
            except (RuntimeError, NotImplementedError) as e:  # pragma: no cover
                pytest.skip(f"torch._scaled_mm not available on this CPU build: {e}")
            d = ulps_apart(bf16_bits(r["out"]), bf16_bits(lib))
            assert d.max() <= 1 and (d != 0).mean() < 0.01, (act_dtype, per_tensor, d.max(), (d != 0).mean())


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_linear_fp8_other_module_dtypes(dtype):
    """fp16 / fp32 modules: per-token rounds to bf16 (bf16 bias) and casts afterwards, per-tensor rounds to the
    module's dtype directly (dax/quant/nn/dynamic/linear.py:106-118, :166-178)."""
    x, w, b = _fp8_case(23, m=48, k=256, n=32)
    x, w, b = x.to(dtype), w.to(dtype), b.to(dtype)
    qw, sw = O.weight_quant_fp8(w)
    r = O.linear_fp8(x, qw, sw, b)
    assert r["out"].dtype == dtype and r["sx"].dtype == torch.float32
    want = scaled_mm_exact(r["xq"].view(torch.uint8).numpy(), 4, qw.view(torch.uint8).numpy(), 4, r["sx"].numpy(), sw.numpy(),
                           bf16_bits(b.bfloat16()))
    d = ulps_apart(bf16_bits(r["out"].bfloat16()), want)  # exact cast back: out holds bf16 values
    assert torch.equal(r["out"], r["out"].bfloat16().to(dtype)) and d.max() <= 1 and (d != 0).mean() < 0.01
    sw1 = O.weight_scale_per_tensor(w, O.E4M3_QMAX)
    qw1 = O.quantize_to_fp8(w, sw1)
    r1 = O.linear_fp8(x, qw1, sw1, b, per_tensor=True)
    acc = decode_fp8(r1["xq"].view(torch.uint8).numpy(), 4) @ decode_fp8(qw1.view(torch.uint8).numpy(), 4).T
    y = acc * float(r1["sx"]) * float(sw1) + b.double().numpy()
    assert r1["out"].dtype == dtype
    rel = np.abs(r1["out"].double().numpy() - y).max() / np.abs(y).max()
    assert rel < (1e-3 if dtype == torch.float16 else 1e-6) and not torch.equal(r1["out"], r1["out"].bfloat16().to(dtype))


def test_float_fallback_rule_and_value():
    """The un-compiled reference hands M <= 16 or K / N not a multiple of 8 to a float matmul on the de-quantised
    weight (dax/quant/nn/dynamic/linear.py:186-202)."""
    assert O.takes_float_fallback(16, 64, 64) and not O.takes_float_fallback(17, 64, 64)
    assert O.takes_float_fallback(64, 60, 64) and O.takes_float_fallback(64, 64, 12) and O.takes_float_fallback(1, 8, 8)
    x, w, b = O.make_inputs(16, 256, 48, seed=31)
    qw, sw = O.weight_quant_int8(w)
    out = O.linear_int8_float_fallback(x, qw, sw, b)
    wd = (qw.bfloat16() * sw.view(-1, 1).bfloat16()).double()  # the weight property: scale and product rounded to bf16
    want = x.double() @ wd.t() + b.double()
    assert out.dtype == torch.bfloat16
    assert float((out.double() - want).norm() / want.norm()) < 4e-3  # bf16 output rounding
    # weight-only quantisation error, against the W8A8 result on the same rows
    q = O.linear_int8(x, qw, sw, b)["out"]
    assert 1e-4 < float((out.float() - q.float()).norm() / q.float().norm()) < 5e-2


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


def test_static_linear_fp8_closed_form_and_library():
    g = torch.Generator().manual_seed(4)
    x = torch.randn(64, 128, generator=g).bfloat16()
    w = (torch.randn(32, 128, generator=g) * 0.05).bfloat16()
    ref0 = torch.nn.functional.linear(x.float(), w.float())
    b = (torch.randn(32, generator=g) * ref0.std()).bfloat16()
    si = O.weight_scale_per_tensor(x, O.E4M3_QMAX)                 # what a MinMaxObserver calibrated on x gives
    sw = O.weight_scale_per_tensor(w, O.E4M3_QMAX)
    qw = O.quantize_to_fp8(w, sw)
    for act_dtype, ebits in ((torch.float8_e4m3fn, 4), (torch.float8_e5m2, 5)):
        si_a = O.weight_scale_per_tensor(x, torch.finfo(act_dtype).max)
        r = O.static_linear_fp8(x, si_a, qw, sw, b, act_dtype)
        want = scaled_mm_exact(r["xq"].view(torch.uint8).numpy(), ebits, qw.view(torch.uint8).numpy(), 4,
                               si_a.numpy().repeat(64), sw.numpy().repeat(32), bf16_bits(b))
        d = ulps_apart(bf16_bits(r["out"]), want)
        assert d.max() <= 1 and (d != 0).mean() < 0.01
        dn = ulps_apart(bf16_bits(O.static_linear_fp8(x, si_a, qw, sw, None, act_dtype)["out"]), want)
        assert (dn != 0).mean() > 0.5  # the bias matters in this case
        # per-tensor scales: the library routine on CPU
        lib = torch._scaled_mm(r["xq"], qw.t(), scale_a=si_a.reshape(()), scale_b=sw.reshape(()), bias=b, out_dtype=torch.bfloat16)
        dl = ulps_apart(bf16_bits(r["out"]), bf16_bits(lib))
        assert dl.max() <= 1 and (dl != 0).mean() < 0.01
    # per-channel weight scale: the same closed form with a scale per column
    qwc, swc = O.weight_quant_e4m3(w)
    rc = O.static_linear_fp8(x, si, qwc, swc, b)
    want = scaled_mm_exact(rc["xq"].view(torch.uint8).numpy(), 4, qwc.view(torch.uint8).numpy(), 4, si.numpy().repeat(64),
                           swc.numpy().reshape(-1), bf16_bits(b))
    d = ulps_apart(bf16_bits(rc["out"]), want)
    assert d.max() <= 1 and (d != 0).mean() < 0.01
    ref = ref0 + b.float()
    assert float((rc["out"].float() - ref).norm() / ref.norm()) < 6e-2    # fp8 (3 mantissa bits) quantisation error


# ------------------------------------------------------------------ general blocks and input dtypes
def test_dynamic_quantize_reduces_to_the_per_row_rule_on_each_block():
    """A block of any shape is the pinned per-row rule applied to the block flattened into one row; the scale
    tensor keeps every reduced dim as 1 in the view shape of the reduction."""
    g = torch.Generator().manual_seed(40)
    x = (torch.randn(2, 6, 8, 12, generator=g) * torch.logspace(-2, 2, 12)).bfloat16()
    x[0, 1] = 0
    assert O.get_reduction_params((3, 3, 2, 10), (3, 3, 10, 10)) == ([3, 3, 5, 2, 10], [0, 1, 3, 4])  # the reference's own example
    cases = {  # block -> scale shape
        (1, 1, 1, 12): (2, 6, 8, 1), (2, 6, 8, 12): (1, 1, 1, 1), (2, 6, 8, 1): (1, 1, 1, 12), (1, 1, 1, 4): (2, 6, 8, 3, 1),
        (1, 3, 2, 12): (2, 2, 1, 4, 1, 1), (2, 1, 8, 6): (1, 6, 1, 2, 1), (1, 6, 1, 1): (2, 1, 8, 12)}
    for target, qmax in ((torch.int8, 127.0), (torch.float8_e4m3fn, 448.0), (torch.float8_e5m2, 57344.0)):
        for block, sshape in cases.items():
            q, sc = O.dynamic_quantize(x, block, target)
            assert q.shape == x.shape and q.dtype == target and sc.dtype == torch.float32 and tuple(sc.shape) == sshape
            qf = q.view(torch.uint8) if target != torch.int8 else q
            # brute force over the blocks
            import itertools
            steps = [range(0, n, b) for n, b in zip(x.shape, block)]
            scs = []
            for origin in itertools.product(*steps):
                sl = tuple(slice(o, o + b) for o, b in zip(origin, block))
                row = x[sl].reshape(1, -1)
                s1 = O.act_scale(row, qmax)
                want = O.quantize_to_int8(row, s1) if target == torch.int8 else O.quantize_to_fp8(row, s1, target).view(torch.uint8)
                assert torch.equal(qf[sl].reshape(1, -1), want), (target, block, origin)
                scs.append(float(s1))
            assert scs == sc.reshape(-1).tolist()  # row-major over the kept dims


def test_act_scale_fp16_and_fp32_inputs_exhaustive():
    """The scale is computed in the input's dtype (dax/quant/nn/dynamic/functional.py:124-129): fp16 rounds the
    quotient to fp16 (subnormals included) before the 2^-23 floor; fp32 does not round."""
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)  # every non-negative finite fp16
    x = torch.from_numpy(h.copy()).view(-1, 1)
    for qmax in (127.0, 448.0, 57344.0):
        got = O.act_scale(x, qmax).view(-1).numpy()
        want = np.maximum((h.astype(np.float32) / np.float32(qmax)).astype(np.float16), np.float16(2.0 ** -23)).astype(np.float32)
        np.testing.assert_array_equal(got, want)
        assert got.min() == np.float32(2.0 ** -23)
    f = (np.random.default_rng(3).standard_normal(5000) * 10.0 ** np.random.default_rng(4).integers(-30, 30, 5000)).astype(np.float32)
    got = O.act_scale(torch.from_numpy(np.abs(f)).view(-1, 1), 127.0).view(-1).numpy()
    np.testing.assert_array_equal(got, np.maximum(np.abs(f) / np.float32(127.0), np.float32(2.0 ** -23)))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_quantize_leaf_other_input_dtypes(closed_form, dtype):
    """x is widened to fp32 exactly before the multiply / divide (fp32 scale), so the closed forms on the fp32
    value hold for fp16 and fp32 inputs; checked through numpy fp32 arithmetic and the C fp8 encoders."""
    g = torch.Generator().manual_seed(41)
    x = (torch.randn(64, 96, generator=g) * torch.logspace(-3, 3, 96)).to(dtype)
    s = O.act_scale(x, 127.0)
    q = O.quantize_to_int8(x, s).numpy()
    inv = (np.float32(1.0) / s.numpy()).astype(np.float32)
    want = np.clip(np.rint((x.float().numpy() * inv).astype(np.float32)), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(q, want)
    for fdt, enc in ((torch.float8_e4m3fn, closed_form.f32_to_e4m3fn), (torch.float8_e5m2, closed_form.f32_to_e5m2)):
        qmax = torch.finfo(fdt).max
        s8 = O.act_scale(x, qmax)
        q8 = O.quantize_to_fp8(x, s8, fdt).view(torch.uint8).numpy()
        v = np.clip((x.float().numpy() / s8.numpy()).astype(np.float32), -qmax, qmax).astype(np.float32)
        np.testing.assert_array_equal(q8, enc(v.reshape(-1)).reshape(v.shape))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_linear_int8_other_module_dtypes(closed_form, dtype):
    """INT8 forward of an fp16 / fp32 module: exact accumulators, fp32 scaling, cast to the module's dtype and a
    bias add in that dtype (dax/quant/nn/dynamic/linear.py:221-228)."""
    x, w, b = O.make_inputs(40, 256, 48, seed=42)
    x, w, b = x.to(dtype), w.to(dtype), b.to(dtype)
    qw, sw = O.weight_quant_int8(w)
    r = O.linear_int8(x, qw, sw, b)
    assert r["out"].dtype == dtype
    acc = closed_form.gemm_i8(r["xq"].numpy(), qw.numpy())
    np.testing.assert_array_equal(r["acc"].numpy(), acc)
    y = (acc.astype(np.float32) * r["sx"].numpy()).astype(np.float32) * sw.numpy()
    npdt = np.float16 if dtype == torch.float16 else np.float32
    want = (y.astype(npdt).astype(np.float32) + b.float().numpy()).astype(npdt)
    np.testing.assert_array_equal(r["out"].numpy(), want)


# ------------------------------------------------------------------ fp32 scale and caller-supplied quant_max / eps / scale_dtype
def _np_bf16_rne(v: np.ndarray) -> np.ndarray:
    """float32 -> nearest bfloat16 (ties to even), returned as float32; finite inputs."""
    u = np.ascontiguousarray(v, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32)


def test_act_scale_fp32_closed_form_exhaustive():
    """act_scale_fp32 = max(f32(amax) / qmax, 2^-23) with an IEEE fp32 division and no rounding to the input's type:
    every non-negative finite bf16 and fp16 abs-max, against numpy float32 arithmetic.  It differs from the eager
    scale on almost every value whose quotient is not a bf16 number."""
    bits = ALL_POS_FINITE = np.arange(0, 0x7F80, dtype=np.uint16)
    a32 = (bits.astype(np.uint32) << 16).view(np.float32)
    xb = from_bits(bits).view(-1, 1)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16)
    xh = torch.from_numpy(h.copy()).view(-1, 1)
    for qmax in (127.0, 448.0, 57344.0):
        got = O.act_scale_fp32(xb, qmax).view(-1).numpy()
        want = np.maximum(a32 / np.float32(qmax), np.float32(2.0 ** -23))
        np.testing.assert_array_equal(got, want)
        eager = O.act_scale(xb, qmax).view(-1).numpy()
        np.testing.assert_array_equal(eager, np.maximum(_np_bf16_rne(a32 / np.float32(qmax)), np.float32(2.0 ** -23)))
        above = want > np.float32(2.0 ** -22)          # (below, both sit on the floor)
        assert (got[above] != eager[above]).mean() > 0.8          # the two forms are different functions (448 = 7 * 64: one quotient in seven is a bf16 number)
        assert (np.abs(got - eager)[above] <= eager[above] * 2.0 ** -8).all()   # ... half a bf16 step apart at most
        goth = O.act_scale_fp32(xh, qmax).view(-1).numpy()
        np.testing.assert_array_equal(goth, np.maximum(h.astype(np.float32) / np.float32(qmax), np.float32(2.0 ** -23)))
    # a row's abs-max decides, sign and position do not; another floor is honoured
    x = torch.tensor([[0.5, -3.0, 2.0], [0.0, 0.0, 0.0]]).bfloat16()
    np.testing.assert_array_equal(O.act_scale_fp32(x, 127.0).view(-1).numpy(), np.array([np.float32(3.0) / np.float32(127.0), 2.0 ** -23], np.float32))
    np.testing.assert_array_equal(O.act_scale_fp32(x, 127.0, eps=0.5).view(-1).numpy(), np.array([0.5, 0.5], np.float32))


def test_fp32_scale_changes_a_small_share_of_the_int8_values():
    """On benchmark-shaped data the fp32 scale moves well under 1 % of the int8 values, each by one step."""
    x, _, _ = O.make_inputs(512, 1536, 8, seed=0)
    q0, s0 = O.act_quant_int8(x)
    q1, s1 = O.act_quant_int8(x, scale_fp32=True)
    assert (s0 != s1).float().mean() > 0.9
    diff = (q0.int() - q1.int()).abs()
    assert int(diff.max()) == 1 and 0.0 < float((diff != 0).float().mean()) < 0.01


def test_dynamic_quantize_with_the_callers_quant_max_eps_and_scale_dtype(closed_form):
    """_dynamic_quantize_func honours quant_max, eps and scale_dtype (dax/quant/nn/dynamic/functional.py:54-61,
    :104-129).  Restated in numpy element by element: abs-max, quotient and floor in x's type; cast to scale_dtype;
    the leaf quantiser rounds 1.0 / scale to the scale's type and the product / quotient to the promoted type of x and
    the scale (bf16 x bf16 -> bf16; bf16 x fp16 or anything with an fp32 side -> fp32)."""
    g = torch.Generator().manual_seed(50)
    x = (torch.randn(48, 64, generator=g) * torch.logspace(-3, 2, 64)).bfloat16()
    x[3] = 0
    xf = x.float().numpy()
    amax = np.abs(xf).max(axis=1, keepdims=True)
    for quant_max, eps in ((127.0, 2.0 ** -23), (100.0, 1e-3), (63, 0.0078125), (448.0, 0.3)):
        s_x = np.maximum(_np_bf16_rne(amax / np.float32(quant_max)), _np_bf16_rne(np.float32([eps])))   # bf16 tensor, bf16 floor
        # fp32 scale: fp32 arithmetic in the leaf quantiser
        q, sc = O.dynamic_quantize(x, (1, 64), torch.int8, quant_max=quant_max, eps=eps, scale_dtype=torch.float32)
        assert sc.dtype == torch.float32
        np.testing.assert_array_equal(sc.numpy(), s_x)
        inv = (np.float32(1.0) / s_x).astype(np.float32)
        np.testing.assert_array_equal(q.numpy(), np.clip(np.rint((xf * inv).astype(np.float32)), -128, 127).astype(np.int8))
        # bf16 scale (scale_dtype=None means x's own type): bf16 arithmetic
        for sd in (torch.bfloat16, None):
            q, sc = O.dynamic_quantize(x, (1, 64), torch.int8, quant_max=quant_max, eps=eps, scale_dtype=sd)
            assert sc.dtype == torch.bfloat16
            np.testing.assert_array_equal(sc.float().numpy(), s_x)
            inv_b = _np_bf16_rne((np.float32(1.0) / s_x).astype(np.float32))
            prod = _np_bf16_rne((xf * inv_b).astype(np.float32))
            np.testing.assert_array_equal(q.numpy(), np.clip(np.rint(prod), -128, 127).astype(np.int8))
        # fp8 with a bf16 scale: the quotient is rounded to bf16 before the clamp and the cast
        for fdt, enc, fmax in ((torch.float8_e4m3fn, closed_form.f32_to_e4m3fn, 448.0), (torch.float8_e5m2, closed_form.f32_to_e5m2, 57344.0)):
            q8, sc8 = O.dynamic_quantize(x, (1, 64), fdt, quant_max=quant_max, eps=eps, scale_dtype=torch.bfloat16)
            np.testing.assert_array_equal(sc8.float().numpy(), s_x)
            v = np.clip(_np_bf16_rne((xf / s_x).astype(np.float32)), -fmax, fmax).astype(np.float32)
            np.testing.assert_array_equal(q8.view(torch.uint8).numpy(), enc(v.reshape(-1)).reshape(v.shape))
        # fp16 scale for a bf16 tensor: the cast can change the value (range); the reciprocal is an fp16 number, the
        # product is promoted to fp32
        q, sc = O.dynamic_quantize(x, (1, 64), torch.int8, quant_max=quant_max, eps=eps, scale_dtype=torch.float16)
        s_h = s_x.astype(np.float16)
        np.testing.assert_array_equal(sc.numpy(), s_h)
        inv = (np.float32(1.0) / s_h.astype(np.float32)).astype(np.float16).astype(np.float32)
        np.testing.assert_array_equal(q.numpy(), np.clip(np.rint((xf * inv).astype(np.float32)), -128, 127).astype(np.int8))
    # the wrappers' defaults are the special case
    q_a, s_a = O.dynamic_quantize(x, (1, 64), torch.int8)
    q_b, s_b = O.dynamic_quantize(x, (1, 64), torch.int8, quant_max=127, eps=torch.finfo(torch.float32).eps, scale_dtype=torch.float32)
    assert torch.equal(q_a, q_b) and torch.equal(s_a, s_b)


def test_scale_by_division_and_by_reciprocal_where_they_differ():
    """torch on a GPU evaluates ``amax / float(quant_max)`` (a tensor over a Python scalar,
    dax/quant/nn/dynamic/functional.py:126) as ``amax * (1 / quant_max)``; on the CPU, and in this build's kernels, it
    is a division.  For bf16 tensors the two give the same scale for every abs-max; for fp16 and fp32 tensors they do
    not always.  This records the deviation set (parity of fp16 / fp32 scales with an eager GPU run is unpinned)."""
    b = (np.arange(0, 0x7F80, dtype=np.uint32) << 16).view(np.float32)
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    counts = {}
    for qmax in (127.0, 448.0, 57344.0):
        r = np.float32(1.0) / np.float32(qmax)
        assert np.array_equal(_np_bf16_rne(b / np.float32(qmax)), _np_bf16_rne((b * r).astype(np.float32)))   # bf16: never
        div = (h / np.float32(qmax)).astype(np.float16)
        mul = (h * r).astype(np.float32).astype(np.float16)
        counts[qmax] = int((div != mul).sum())
    assert counts[127.0] == 0 and 0 < counts[448.0] < 100 and 0 < counts[57344.0] < 100   # fp16: a few dozen of 31 744 values
    f = np.abs(np.random.default_rng(7).standard_normal(200000).astype(np.float32)) * np.float32(3.0)
    for qmax, lo, hi in ((127.0, 0.01, 0.15), (448.0, 0.3, 0.7)):
        r = np.float32(1.0) / np.float32(qmax)
        share = float(((f / np.float32(qmax)) != (f * r).astype(np.float32)).mean())
        assert lo < share < hi, (qmax, share)       # fp32: a few percent at 127, about half at 448, each one ulp
        assert np.abs((f / np.float32(qmax)).view(np.int32) - (f * r).astype(np.float32).view(np.int32)).max() <= 1
