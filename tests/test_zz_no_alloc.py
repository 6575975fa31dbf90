"""The split-K linear on the library's own scratch array (daxq_linear_w8a8_splitk_static): an entry point that
allocates nothing.  Called through the C ABI and compared, bit for bit, with daxq_linear_w8a8_splitk on a caller
workspace and with the oracle, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest
import torch

from oracle import daxq_oracle as O
from tests.util import bf16_bits

pytestmark = pytest.mark.gpu


def dev(t):
    return t.to("cuda") if t is not None else None


def _call_static(L, fmt, xq, sx, wq, sw, b, out, splits):
    m, k = xq.shape
    n = wq.shape[0]
    st = torch.cuda.current_stream().cuda_stream
    return L.daxq_linear_w8a8_splitk_static(fmt, fmt, xq.data_ptr(), xq.stride(0), sx.data_ptr(), wq.data_ptr(), wq.stride(0),
                                            sw.data_ptr(), b.data_ptr() if b is not None else None, out.data_ptr(), n, m, n, k,
                                            splits, st)


def _call_workspace(L, fmt, xq, sx, wq, sw, b, out, splits, ws):
    m, k = xq.shape
    n = wq.shape[0]
    st = torch.cuda.current_stream().cuda_stream
    return L.daxq_linear_w8a8_splitk(fmt, fmt, xq.data_ptr(), xq.stride(0), sx.data_ptr(), wq.data_ptr(), wq.stride(0),
                                     sw.data_ptr(), b.data_ptr() if b is not None else None, out.data_ptr(), n, m, n, k,
                                     splits, ws.data_ptr(), ws.numel(), st)


def test_static_scratch_splitk_equals_workspace_form_two_calls_in_a_row():
    import dax_amd.ops as ops
    from dax_amd import _capi

    L = _capi.lib()
    ws = torch.zeros(40 << 20, dtype=torch.uint8, device="cuda")
    # the second call is smaller than the first (fewer tiles, fewer ranges): it finds the first call's partial
    # results in the array and counters that the first call set back to zero
    for m, n, k, splits in [(512, 5120, 5120, 2), (300, 640, 1024, 4), (256, 5120, 5120, 0)]:
        x, w, b = O.make_inputs(m, k, n, seed=m + k)
        qw, sw = O.weight_quant_int8(w)
        ref = O.linear_int8(x, qw, sw, b, keep_acc=False)["out"]
        xq, sx = ops.act_quant_i8(dev(x))
        wq_d, sw_d, b_d = dev(qw), dev(sw.view(-1)), dev(b)
        out_s = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        out_w = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        assert _call_static(L, 0, xq, sx, wq_d, sw_d, b_d, out_s, splits) == 0, _capi.last_error()
        assert _call_workspace(L, 0, xq, sx, wq_d, sw_d, b_d, out_w, splits, ws) == 0, _capi.last_error()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bf16_bits(out_s), bf16_bits(out_w), err_msg=str((m, n, k, splits)))
        np.testing.assert_array_equal(bf16_bits(out_s), bf16_bits(ref), err_msg=str((m, n, k, splits)))


def test_static_scratch_splitk_fp8_and_limits():
    import dax_amd.ops as ops
    from dax_amd import _capi

    L = _capi.lib()
    ws = torch.zeros(40 << 20, dtype=torch.uint8, device="cuda")
    for m, n, k, splits in [(512, 1536, 2048, 4), (256, 512, 1024, 2)]:
        x, w, b = O.make_inputs(m, k, n, seed=7 + m)
        qw, sw = O.weight_quant_e4m3(w)
        xq, sx = ops.act_quant_e4m3(dev(x))
        wq_d, sw_d, b_d = dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b)
        out_s = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        out_w = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        assert _call_static(L, 1, xq, sx, wq_d, sw_d, b_d, out_s, splits) == 0, _capi.last_error()
        assert _call_workspace(L, 1, xq, sx, wq_d, sw_d, b_d, out_w, splits, ws) == 0, _capi.last_error()
        torch.cuda.synchronize()
        assert torch.equal(out_s, out_w)     # same kernels, partial sums added in range order
    # beyond the array: 40 x 40 tiles in 2 ranges = 3200 partial results; rejected before any launch
    xq = torch.zeros(5120, 1024, dtype=torch.int8, device="cuda")
    wq = torch.zeros(5120, 1024, dtype=torch.int8, device="cuda")
    one = torch.ones(5120, device="cuda")
    out = torch.full((5120, 5120), 3.0, dtype=torch.bfloat16, device="cuda")
    rc = _call_static(L, 0, xq, one, wq, one, None, out, 2)
    assert rc == -1 and "scratch" in _capi.last_error()
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
    # splits = 1 (and the library's choice for a launch with enough tiles) is the plain launch
    assert _call_static(L, 0, xq, one, wq, one, None, out, 0) == 0
    torch.cuda.synchronize()
    assert bool((out == 0).all())
