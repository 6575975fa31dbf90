"""GPU parity of the HIP quantisers against the oracle, through torch.ops.daxq -> C ABI.

Integer / byte outputs and scales are compared bit for bit.
"""
import numpy as np
import pytest
import torch

from oracle import daxq_oracle as O
from tests.util import ALL_POS_FINITE, FINITE_BF16, from_bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import dax_amd.ops as ops

    return ops


def dev(t):
    return t.to("cuda")


def test_device_is_gfx950():
    from dax_amd import _capi

    info = _capi.device_info(0)
    assert info["status"] == 0 and info["arch"].startswith("gfx950"), info
    print("device:", info)


SHAPES = [(64, 384), (130, 1536), (33, 5120), (17, 13824), (5, 8960), (7, 200), (3, 100), (1, 8), (2, 7),
          (9, 18432), (4, 20480), (300, 128)]


@pytest.mark.parametrize("m,k", SHAPES)
def test_act_quant_i8_matches_oracle(ops, m, k):
    x, _, _ = O.make_inputs(m, k, 8, seed=m * 7 + k)
    if m > 2:
        x[1] = 0                      # zero row -> scale 2^-23, all zeros
        x[2] = 0
        x[2, k // 2] = -3e-30         # below the eps floor
    q, s = ops.act_quant_i8(dev(x))
    torch.cuda.synchronize()
    qo, so = O.act_quant_int8(x)
    kp = ops.pad_k(k)
    assert q.shape == (m, kp) and q.dtype == torch.int8 and s.shape == (m,)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    np.testing.assert_array_equal(q[:, :k].cpu().numpy(), qo.numpy())
    assert not q[:, k:].any()         # K padding is zero


@pytest.mark.parametrize("m,k", SHAPES)
def test_act_quant_e4m3_matches_oracle(ops, m, k):
    x, _, _ = O.make_inputs(m, k, 8, seed=m * 11 + k)
    if m > 2:
        x[1] = 0
    q, s = ops.act_quant_e4m3(dev(x))
    torch.cuda.synchronize()
    qo, so = O.act_quant_e4m3(x)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    np.testing.assert_array_equal(q[:, :k].cpu().numpy(), qo.view(torch.uint8).numpy())
    assert not q[:, k:].any()


@pytest.mark.parametrize("m,k", SHAPES)
def test_act_quant_e5m2_matches_oracle(ops, m, k):
    x, _, _ = O.make_inputs(m, k, 8, seed=m * 13 + k)
    if m > 2:
        x[1] = 0
    q, s = ops.act_quant_e5m2(dev(x))
    torch.cuda.synchronize()
    qo, so = O.act_quant_e5m2(x)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    np.testing.assert_array_equal(q[:, :k].cpu().numpy(), qo.view(torch.uint8).numpy())
    assert not q[:, k:].any()


def test_act_quant_e5m2_every_bf16_amax_and_value(ops):
    # rows: every finite bf16 value once as the row abs-max (alternating sign), and a second block
    # where every finite bf16 value appears under a large fixed abs-max
    n = ALL_POS_FINITE.size
    x = torch.zeros(n, 64, dtype=torch.bfloat16)
    vals = from_bits(ALL_POS_FINITE)
    sign = torch.where(torch.arange(n) % 2 == 1, -1.0, 1.0).bfloat16()
    x[torch.arange(n), torch.arange(n) % 64] = vals * sign
    allv = from_bits(FINITE_BF16).view(-1, 64)            # 1020 rows of 64 distinct values
    xs = torch.cat([x, allv])
    q, s = ops.act_quant_e5m2(dev(xs))
    qo, so = O.act_quant_e5m2(xs)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    np.testing.assert_array_equal(q[:, :64].cpu().numpy(), qo.view(torch.uint8).numpy())


def test_act_quant_strided_rows(ops):
    x, _, _ = O.make_inputs(40, 512, 8, seed=5)
    big = torch.zeros(40, 640, dtype=torch.bfloat16)
    big[:, :512] = x
    xs = dev(big)[:, :512]            # row stride 640
    q, s = ops.act_quant_i8(xs)
    qo, so = O.act_quant_int8(x)
    np.testing.assert_array_equal(q[:, :512].cpu().numpy(), qo.numpy())
    np.testing.assert_array_equal(s.cpu().numpy(), so.view(-1).numpy())


@pytest.mark.parametrize("fp8", [False, True])
def test_act_scale_exhaustive_every_bf16_amax(ops, fp8):
    # one row per amax value; the amax sits in a different column each row, negative on odd rows
    n = ALL_POS_FINITE.size
    x = torch.zeros(n, 64, dtype=torch.bfloat16)
    vals = from_bits(ALL_POS_FINITE)
    cols = torch.arange(n) % 64
    sign = torch.where(torch.arange(n) % 2 == 1, -1.0, 1.0).bfloat16()
    x[torch.arange(n), cols] = vals * sign
    q, s = (ops.act_quant_e4m3 if fp8 else ops.act_quant_i8)(dev(x))
    qo, so = (O.act_quant_e4m3 if fp8 else O.act_quant_int8)(x)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    qo_b = qo.view(torch.uint8).numpy() if fp8 else qo.numpy()
    np.testing.assert_array_equal(q[:, :64].cpu().numpy(), qo_b)


@pytest.mark.parametrize("fmt", ["e4m3", "e5m2"])
def test_dynamic_fp8_division_every_bf16_value_under_sampled_abs_max(ops, fmt):
    """The dynamic FP8 quantiser divides through the row's reciprocal with an exact fma correction instead of a
    spelled-out division: every finite bf16 value that fits under a row abs-max, for 640 abs-max values spread over
    all exponents (both signs), must still give the bytes of the reference's true division."""
    rng = np.random.default_rng(11)
    amax_bits = np.unique(np.concatenate([rng.choice(ALL_POS_FINITE[1:], 600, replace=False),
                                          ALL_POS_FINITE[-20:], ALL_POS_FINITE[1:21]]))
    allv = from_bits(FINITE_BF16)                                   # 65280 values
    chunks = allv.view(-1, 16320)                                   # 4 x 16320
    rows = []
    for ab in amax_bits:
        a = from_bits(np.array([ab], dtype=np.uint16))
        body = torch.where(chunks.float().abs() <= a.float(), chunks, torch.zeros_like(chunks))
        head = torch.zeros(4, 8, dtype=torch.bfloat16)
        head[:, 0] = a if ab % 2 == 0 else -a
        rows.append(torch.cat([head, body], 1))                     # 4 rows of 16328 (wave kernel: row in registers)
    x = torch.cat(rows)
    fn, ofn = (ops.act_quant_e4m3, O.act_quant_e4m3) if fmt == "e4m3" else (ops.act_quant_e5m2, O.act_quant_e5m2)
    q, s = fn(dev(x))
    qo, so = ofn(x)
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), so.view(-1).numpy().view(np.uint32))
    bad = int((q[:, :x.shape[1]].cpu() != qo.view(torch.uint8)).sum())
    assert bad == 0, f"{bad} of {x.numel()} bytes differ"
    # the general (one block per row) kernel takes the same formula: rows too long for the register kernel
    xl = x.view(-1, 4 * 16328)[:40].contiguous()
    q2, s2 = fn(dev(xl))
    qo2, so2 = ofn(xl)
    assert torch.equal(q2[:, :xl.shape[1]].cpu(), qo2.view(torch.uint8)) and torch.equal(s2.cpu(), so2.view(-1))


def _sampled_scales(qmax, n_act, n_f32, seed):
    x = from_bits(ALL_POS_FINITE).view(-1, 1)
    reach = np.unique(O.act_scale(x, qmax).view(-1).numpy())
    rng = np.random.default_rng(seed)
    act = np.concatenate([reach[:3], reach[-3:], rng.choice(reach, n_act, replace=False)])
    # un-rounded fp32 scales as the weight path produces them
    f32 = np.exp(rng.uniform(np.log(1e-6), np.log(10.0), n_f32)).astype(np.float32)
    return np.concatenate([act, f32]).astype(np.float32)


@pytest.mark.parametrize("fp8", [False, True])
def test_leaf_quantiser_every_bf16_x_many_scales(ops, fp8):
    # rows = scales, columns = every finite bf16 value: 65280 x 384 = 25 M (x, scale) pairs
    scales = _sampled_scales(448.0 if fp8 else 127.0, 250, 128, seed=3)
    xrow = from_bits(FINITE_BF16)
    x = xrow.view(1, -1).expand(scales.size, -1).contiguous()
    st = torch.from_numpy(scales)
    fn = ops.quantize_rows_e4m3 if fp8 else ops.quantize_rows_i8
    q = fn(dev(x), dev(st)).cpu()
    if fp8:
        want = O.quantize_to_fp8(x, st.view(-1, 1)).view(torch.uint8)
    else:
        want = O.quantize_to_int8(x, st.view(-1, 1))
    assert torch.equal(q, want), f"{(q != want).sum().item()} mismatches"


@pytest.mark.parametrize("qmax", [127.0, 448.0])
def test_weight_observer_kernels(ops, qmax):
    _, w, _ = O.make_inputs(4, 1000, 300, seed=8)
    w[3] = 0
    w[4, 0] = -2.0
    w[5] = w[5].abs()                 # all-positive row: -min < 0
    w[6] = -w[6].abs() - 0.01         # all-negative row
    lo, hi = ops.row_minmax(dev(w))
    lo_o, hi_o = torch.aminmax(w.float(), dim=1)
    assert torch.equal(lo.cpu(), lo_o) and torch.equal(hi.cpu(), hi_o)
    s = ops.scale_from_minmax(lo, hi, qmax).cpu()
    so = O.weight_scale(w, qmax)
    np.testing.assert_array_equal(s.numpy().view(np.uint32), so.numpy().view(np.uint32))


@pytest.mark.parametrize("k,ld_q", [(200, 512), (5120, 5248), (7, 300), (384, 384), (1000, 1008)])
def test_quantisers_leave_a_wider_row_stride_alone(ops, k, ld_q):
    """Through the C ABI with a row stride beyond the padded row: values in [0, k), zeros up to the next multiple of
    128 (as far as the row reaches), and not a byte touched behind that (the output may be a column slice of a wider
    buffer, or rows kept apart on purpose)."""
    from dax_amd import _capi

    L = _capi.lib()
    m = 37
    x, _, _ = O.make_inputs(m, k, 8, seed=k)
    xd = dev(x)
    st = torch.cuda.current_stream().cuda_stream
    kp = min(ld_q, (k + 127) // 128 * 128)
    ref_q, ref_s = O.act_quant_int8(x)
    for fn, extra in ((L.daxq_act_quant_i8, ()), (L.daxq_gelu_tanh_act_quant_i8, None)):
        q = torch.full((m, ld_q), 0x55, dtype=torch.int8, device="cuda")
        s = torch.zeros(m, device="cuda")
        if extra is None:
            if k % 8:
                continue           # the fused producers take rows of whole 16-byte pieces only
            rc = fn(xd.data_ptr(), m, k, k, None, 0, q.data_ptr(), ld_q, s.data_ptr(), st)
        else:
            rc = fn(xd.data_ptr(), m, k, k, q.data_ptr(), ld_q, s.data_ptr(), st)
        assert rc == 0, _capi.last_error()
        torch.cuda.synchronize()
        assert bool((q[:, k:kp] == 0).all()) and bool((q[:, kp:] == 0x55).all())
        if extra is not None:
            assert torch.equal(q[:, :k].cpu(), ref_q[:, :k]) and torch.equal(s.cpu(), ref_s.view(-1))


def test_activation_rows_of_whole_kilobytes_are_kept_apart(ops):
    """Quantised activations whose rows are a multiple of 1 KB long come back with a row stride 128 bytes larger
    (memory channels, see ops.Q_ROW_PAD); the GEMM follows the stride, values and results are the oracle's."""
    m, k, n = 300, 1024, 256
    x, w, b = O.make_inputs(m, k, n, seed=3)
    qw, sw = O.weight_quant_int8(w)
    ref = O.linear_int8(x, qw, sw, b)
    xq, sx = ops.act_quant_i8(dev(x))
    assert xq.shape == (m, k) and xq.stride() == (k + 128, 1)
    assert torch.equal(xq.cpu(), ref["xq"])
    out = ops.linear_i8(xq, sx, dev(qw), dev(sw.view(-1)), dev(b))
    assert torch.equal(out.cpu().view(torch.int16), ref["out"].view(torch.int16))
    xq2, _ = ops.act_quant_i8(dev(x[:, :896].contiguous()))
    assert xq2.stride() == (896, 1)          # 7 x 128: not a multiple of 1 KB, rows contiguous
    q3, _, _ = ops.gelu_tanh_act_quant_i8(dev(x))
    assert q3.shape == (m, k) and q3.stride() == (k + 128, 1)


def test_cpu_tensor_is_rejected_loudly(ops):
    with pytest.raises((RuntimeError, NotImplementedError)):
        ops.act_quant_i8(torch.zeros(4, 128, dtype=torch.bfloat16))
