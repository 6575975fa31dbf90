"""daxq_dynamic_linear*: quantiser + GEMM behind one C entry point, called through raw ctypes on caller-owned buffers
and compared with the oracle's forward of the dynamic linear (dax/quant/nn/dynamic/linear.py:146-228).

INT8: quantised bytes, scales and bf16 outputs bit for bit; FP8: bytes and scales bit for bit, outputs within the stated
2e-2 relative L2 (observed ~2e-3).  Also: nothing outside the rows / columns the call owns is written, and the op the
module calls (torch.ops.daxq.dynamic_linear_*) returns the same bits as the two separate ops.
"""
import numpy as np
import pytest
import torch

from oracle import daxq_oracle as O
from tests.util import bf16_bits, rel_l2

pytestmark = pytest.mark.gpu

FP8_TOL = 2e-2


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _pad128(k):
    return (k + 127) // 128 * 128


def _weights(w, fmt):
    """oracle weight quantisation -> (bytes [N, pad128(K)] on the device, fp32 scales [N] on the device, cpu pair)"""
    qw, sw = (O.weight_quant_int8 if fmt == "i8" else O.weight_quant_e4m3)(w)
    n, k = w.shape
    kp = _pad128(k)
    raw = qw if fmt == "i8" else qw.view(torch.uint8)
    wide = torch.zeros((n, kp), dtype=raw.dtype, device="cuda")
    wide[:, :k] = raw.to("cuda")
    return wide, sw.reshape(-1).float().to("cuda"), (qw, sw)


SHAPES = [(300, 520, 256), (4096, 1536, 1536), (17, 264, 384), (1, 128, 128), (700, 392, 200), (130, 130, 1000),
          (512, 5120, 5120), (64, 24, 136)]


@pytest.mark.parametrize("named", [False, True])
@pytest.mark.parametrize("m,n,k", SHAPES)
def test_dynamic_linear_i8_through_the_c_abi_bit_exact(m, n, k, named):
    from dax_amd import _capi

    L = _capi.lib()
    x, w, b = O.make_inputs(m, k, n, seed=m + n + k)
    wq, sw, (qw_cpu, sw_cpu) = _weights(w, "i8")
    ref = O.linear_int8(x, qw_cpu, sw_cpu, b)
    kp, pad = _pad128(k), 64
    rows = m if named else max(m, 128)
    xd, bd = x.to("cuda"), b.to("cuda")
    xq = torch.full((rows + 1, kp + pad), 9, dtype=torch.int8, device="cuda")
    sx = torch.full((rows + 1,), -3.0, dtype=torch.float32, device="cuda")
    out = torch.full((rows + 1, n + 8), 5.0, dtype=torch.bfloat16, device="cuda")
    if named:
        rc = L.daxq_dynamic_linear_i8(xd.data_ptr(), k, xq.data_ptr(), kp + pad, sx.data_ptr(), wq.data_ptr(), kp, sw.data_ptr(),
                                      bd.data_ptr(), out.data_ptr(), n + 8, m, n, k, _stream())
    else:
        rc = L.daxq_dynamic_linear(0, 0, 0, 0, 1, xd.data_ptr(), k, xq.data_ptr(), kp + pad, sx.data_ptr(), rows, wq.data_ptr(), kp,
                                   sw.data_ptr(), bd.data_ptr(), out.data_ptr(), n + 8, m, n, k, None, 0, 0, _stream())
    _capi.check(rc, "dynamic_linear_i8")
    torch.cuda.synchronize()
    assert torch.equal(xq[:m, :k].cpu(), ref["xq"])
    assert bool((xq[:m, k:kp] == 0).all()) and bool((xq[:m, kp:] == 9).all())
    assert torch.equal(sx[:m].cpu(), ref["sx"].reshape(-1))
    np.testing.assert_array_equal(bf16_bits(out[:m, :n]), bf16_bits(ref["out"]))
    # nothing beyond the buffers' own rows and columns is written
    assert bool((xq[rows:] == 9).all()) and bool((sx[rows:] == -3.0).all())
    assert bool((out[rows:] == 5.0).all()) and bool((out[:, n:] == 5.0).all())
    if rows == m:
        assert bool((xq[m:] == 9).all()) and bool((out[m:] == 5.0).all())


@pytest.mark.parametrize("x_fmt", ["e4m3", "e5m2"])
@pytest.mark.parametrize("m,n,k", SHAPES[:6])
def test_dynamic_linear_fp8_through_the_c_abi(m, n, k, x_fmt):
    from dax_amd import _capi

    L = _capi.lib()
    x, w, b = O.make_inputs(m, k, n, seed=3 * m + n + k)
    wq, sw, (qw_cpu, sw_cpu) = _weights(w, "e4m3")
    act = torch.float8_e5m2 if x_fmt == "e5m2" else torch.float8_e4m3fn
    ref = O.linear_e4m3(x, qw_cpu, sw_cpu, b, act_dtype=act)
    kp = _pad128(k)
    xd, bd = x.to("cuda"), b.to("cuda")
    xq = torch.full((m, kp), 1, dtype=torch.uint8, device="cuda")
    sx = torch.zeros((m,), dtype=torch.float32, device="cuda")
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    fn = L.daxq_dynamic_linear_e5m2_e4m3 if x_fmt == "e5m2" else L.daxq_dynamic_linear_e4m3
    _capi.check(fn(xd.data_ptr(), k, xq.data_ptr(), kp, sx.data_ptr(), wq.data_ptr(), kp, sw.data_ptr(), bd.data_ptr(),
                   out.data_ptr(), n, m, n, k, _stream()), "dynamic_linear_" + x_fmt)
    torch.cuda.synchronize()
    assert torch.equal(xq[:, :k].cpu(), ref["xq"].view(torch.uint8))
    assert torch.equal(sx.cpu(), ref["sx"].reshape(-1))
    assert rel_l2(out, ref["out"]) < FP8_TOL


def test_dynamic_linear_with_a_split_k_workspace_bit_exact():
    """M = 256, N = K = 5120 with a caller workspace: K is cut into ranges, and the outputs are the plain launch's bits."""
    from dax_amd import _capi

    L = _capi.lib()
    m, n, k = 256, 5120, 5120
    splits = L.daxq_linear_splitk_choice(m, n, k)
    assert splits > 1
    x, w, b = O.make_inputs(m, k, n, seed=5)
    wq, sw, (qw_cpu, sw_cpu) = _weights(w, "i8")
    ref = O.linear_int8(x, qw_cpu, sw_cpu, b)
    xd, bd = x.to("cuda"), b.to("cuda")
    need = L.daxq_linear_splitk_workspace_bytes(m, n, splits)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    for workspace in (ws, None):
        xq = torch.empty((m, k), dtype=torch.int8, device="cuda")
        sx = torch.empty((m,), dtype=torch.float32, device="cuda")
        out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
        _capi.check(L.daxq_dynamic_linear(0, 0, 0, 0, 1, xd.data_ptr(), k, xq.data_ptr(), k, sx.data_ptr(), m, wq.data_ptr(), k,
                                          sw.data_ptr(), bd.data_ptr(), out.data_ptr(), n, m, n, k,
                                          workspace.data_ptr() if workspace is not None else None,
                                          workspace.numel() if workspace is not None else 0, 0, _stream()), "dynamic_linear")
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref["out"]))
    assert bool((ws[:16384] == 0).all())  # the counters are left at zero


def test_dynamic_linear_rejects_bad_arguments():
    from dax_amd import _capi

    L = _capi.lib()
    t = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = t.data_ptr()
    # rows_alloc < m, a leading dimension that does not reach the padded K, mixed operand formats
    assert L.daxq_dynamic_linear(0, 0, 0, 0, 1, p, 128, p, 128, p, 1, p, 128, p, None, p, 8, 2, 8, 128, None, 0, 0, _stream()) == -1
    assert L.daxq_dynamic_linear(0, 0, 0, 0, 1, p, 100, p, 100, p, 2, p, 128, p, None, p, 8, 2, 8, 100, None, 0, 0, _stream()) == -1
    assert L.daxq_dynamic_linear(0, 0, 1, 0, 1, p, 128, p, 128, p, 2, p, 128, p, None, p, 8, 2, 8, 128, None, 0, 0, _stream()) == -1
    assert "dynamic_linear" in _capi.last_error() or "unsupported operand formats" in _capi.last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize("fmt", ["i8", "e4m3", "e5m2"])
@pytest.mark.parametrize("m,n,k", [(300, 520, 256), (5, 264, 384), (4096, 1536, 1536), (256, 5120, 5120)])
def test_fused_op_equals_the_two_ops(m, n, k, fmt):
    """torch.ops.daxq.dynamic_linear_* (one C call, two allocations) against act_quant_* followed by linear_*."""
    import dax_amd.ops as ops

    x, w, b = O.make_inputs(m, k, n, seed=11 + m)
    wq, sw, _ = _weights(w, "i8" if fmt == "i8" else "e4m3")
    xd, bd = x.to("cuda"), b.to("cuda")
    fused = {"i8": ops.dynamic_linear_i8, "e4m3": ops.dynamic_linear_e4m3, "e5m2": ops.dynamic_linear_e5m2_e4m3}[fmt]
    quant = {"i8": ops.act_quant_i8, "e4m3": ops.act_quant_e4m3, "e5m2": ops.act_quant_e5m2}[fmt]
    lin = {"i8": ops.linear_i8, "e4m3": ops.linear_e4m3, "e5m2": ops.linear_e5m2_e4m3}[fmt]
    got = fused(xd, wq, sw, bd)
    xq, sx = quant(xd)
    want = lin(xq, sx, wq, sw, bd)
    torch.cuda.synchronize()
    assert got.shape == (m, n)
    if fmt == "i8" or m >= 128:
        np.testing.assert_array_equal(bf16_bits(got), bf16_bits(want))
    else:  # fewer than 128 rows: the fused op runs the tiled kernel, the separate ops the generic one (fp32 summation order)
        assert rel_l2(got, want) < 2e-3


def test_prepared_forward_follows_replaced_state():
    """The swapped module keeps its GEMM operands ready between forwards.  State that is replaced afterwards -- by
    assignment, behind the module's back in its buffer / parameter tables (as off-loading hooks do), through `.data`,
    or updated in place -- must be what the next forward computes with."""
    from torch import nn

    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    m, k, n = 200, 256, 384
    x, w, b = O.make_inputs(m, k, n, seed=91)
    _, w2, b2 = O.make_inputs(m, k, n, seed=92)
    lin = nn.Linear(k, n).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    model = nn.Sequential(lin).to("cuda")
    quantize_dynamic(model, {"": cfg()})
    q = model[0]
    xd = x.to("cuda")

    def check(wt, bt, what):
        qw, sw = O.weight_quant_int8(wt)
        ref = O.linear_int8(x, qw, sw, bt)["out"]
        with torch.no_grad():
            got = q(xd)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bf16_bits(got), bf16_bits(ref), err_msg=what)

    check(w, b, "as converted")
    assert q._fast is not None
    qw2, sw2 = O.weight_quant_int8(w2)
    with torch.no_grad():
        q.bias.copy_(b2.to("cuda"))                      # in place
    check(w, b2, "bias updated in place")
    q.bias.data = b.to("cuda").clone()                   # through .data
    check(w, b, "bias replaced through .data")
    q.qweight = qw2.to("cuda")                           # by assignment
    q.weight_scale = sw2.reshape(1, -1).to("cuda")
    check(w2, b, "qweight and weight_scale assigned")
    qw1, sw1 = O.weight_quant_int8(w)
    q._buffers["qweight"] = qw1.to("cuda")               # behind the module's back
    q._buffers["weight_scale"] = sw1.reshape(1, -1).to("cuda")
    q._parameters["bias"] = nn.Parameter(b2.to("cuda"))
    check(w, b2, "state tables replaced directly")
    with torch.no_grad():
        q.qweight.copy_(qw2.to("cuda"))                  # in place
        q.weight_scale.copy_(sw2.reshape(1, -1).to("cuda"))
    check(w2, b2, "qweight updated in place")
    x3 = x.view(2, 100, k).to("cuda")
    with torch.no_grad():
        got3 = q(x3)
    assert got3.shape == (2, 100, n)
    ref3 = O.linear_int8(x, qw2, sw2, b2)["out"]
    np.testing.assert_array_equal(bf16_bits(got3.reshape(m, n)), bf16_bits(ref3))
