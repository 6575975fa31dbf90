"""Parity at the exact shapes of the five benchmark configurations (config 0: M=4096, K=N=1536; 1: Wan 1.3B 480p; 2 / 3: Wan 14B 720p INT8 / FP8; 4: the 40-layer set),
through the swapped module.  Rows of a per-token-quantised linear are independent, so at the large M a
sample of rows (first / last rows of the first / last tiles plus random ones) is compared with the
oracle bit for bit (INT8) or within 2e-2 relative L2 (FP8), and the whole output is tied to it by
running the same module on the row sample alone: the two GPU results must be identical, INT8 and FP8 alike (a token's
output does not depend on the batch it arrives in)."""
import numpy as np
import pytest
import torch
from torch import nn

from oracle import daxq_oracle as O
from tests.util import bf16_bits, rel_l2

pytestmark = pytest.mark.gpu
FP8_TOL = 2e-2


def _quantised(k, n, w, b, fp8):
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig as f8,
                                                    get_dynamic_int8_per_token_act_per_channel_weight_qconfig as i8)

    lin = nn.Linear(k, n).bfloat16()
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    model = nn.Sequential(lin).to("cuda")
    quantize_dynamic(model, {"": f8(activation_dtype=torch.float8_e4m3fn) if fp8 else i8()})
    return model[0]


def _rows(m, extra=160, seed=0):
    edge = [r for r in (0, 1, 127, 128, 255, 256, 257, m - 257, m - 256, m - 129, m - 2, m - 1) if 0 <= r < m]
    g = torch.Generator().manual_seed(seed)
    return torch.cat([torch.tensor(edge), torch.randint(0, m, (extra,), generator=g)]).unique()


def _check(m, k, n, seed, fp8, x=None):
    xs, w, b = O.make_inputs(m if x is None else 8, k, n, seed=seed)
    if x is None:
        x = xs
    q = _quantised(k, n, w, b, fp8)
    xd = x.to("cuda")
    y = q(xd)
    assert y.shape == (m, n) and y.dtype == torch.bfloat16
    rows = _rows(m)
    y_rows = q(xd[rows.to("cuda")].contiguous())
    # (FP8 too: every tile size, tile order and launch cut runs the same sequence of MFMAs per output element)
    assert torch.equal(y[rows.to("cuda")], y_rows), "full-M launch and row-sample launch disagree"
    if fp8:
        qw, sw = O.weight_quant_e4m3(w)
        ref = O.linear_e4m3(x[rows], qw, sw, b)["out"]
        assert torch.equal(q.qweight.cpu().view(torch.uint8), qw.view(torch.uint8))
        assert rel_l2(y_rows, ref) < FP8_TOL
    else:
        qw, sw = O.weight_quant_int8(w)
        ref = O.linear_int8(x[rows], qw, sw, b, keep_acc=False)["out"]
        assert torch.equal(q.qweight.cpu(), qw) and torch.equal(q.weight_scale.cpu(), sw)
        np.testing.assert_array_equal(bf16_bits(y_rows), bf16_bits(ref))
    return y


def test_config0_int8_whole_output():
    # config 0: M=4096, K=N=1536, seed 0 -- every element against the oracle
    m, k, n = 4096, 1536, 1536
    x, w, b = O.make_inputs(m, k, n, seed=0)
    q = _quantised(k, n, w, b, False)
    y = q(x.to("cuda"))
    qw, sw = O.weight_quant_int8(w)
    ref = O.linear_int8(x, qw, sw, b, keep_acc=False)["out"]
    np.testing.assert_array_equal(bf16_bits(y), bf16_bits(ref))
    # and against the float layer it replaces (quantisation error, not a parity bound)
    fl = torch.nn.functional.linear(x.float(), w.float(), b.float())
    assert rel_l2(y, fl) < 5e-2


@pytest.mark.parametrize("k,n", [(1536, 4608), (1536, 1536), (1536, 8960), (8960, 1536)])
def test_config1_wan_1_3b_480p_shapes(k, n):
    _check(32760, k, n, seed=1, fp8=False)          # 32760 = 127 * 256 + 248: ragged last tile


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("k,n", [(5120, 15360), (5120, 13824), (13824, 5120)])
def test_config2_3_wan_14b_720p_shapes(k, n, fp8):
    # (the 5120 -> 5120 out-projection is covered in test_gpu_linear.py, with accumulators)
    _check(75600, k, n, seed=2, fp8=fp8)


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("m,k,n", [(1100, 2048, 4352), (1024, 5120, 5120)])
def test_mid_size_launches_on_half_tiles(m, k, n, fp8):
    """Between a quarter and a half of 256 CUs' worth of 256x256 tiles (85 and 80 here, K >= 2048) the library runs every
    tile as its two 256x128 halves: outputs against the oracle, and the same bits as the launch of a row sample, which
    takes the 128x128 tiles."""
    tiles = -(-m // 256) * -(-n // 256)
    assert 64 < tiles <= 128 and k >= 2048
    _check(m, k, n, seed=5, fp8=fp8)


def test_config4_cross_attention_small_m():
    # K / V projections of the 512-token text context (skinny M), and M = 1 / 17 leftovers
    for m in (512, 17, 1):
        x, w, b = O.make_inputs(m, 5120, 5120, seed=4)
        q = _quantised(5120, 5120, w, b, False)
        y = q(x.to("cuda"))
        qw, sw = O.weight_quant_int8(w)
        ref = O.linear_int8(x, qw, sw, b, keep_acc=False)["out"]
        np.testing.assert_array_equal(bf16_bits(y), bf16_bits(ref))


@pytest.mark.parametrize("fp8", [False, True])
def test_fewer_rows_than_a_tile(fp8):
    """M below 128: the module quantises into a 128-row buffer and runs the tiled kernel on it (the rows beyond M hold
    whatever the allocation held); the result has M rows, is contiguous, views like any other, and equals the oracle
    (INT8 bit for bit).  Shapes that the generic kernel still takes (N < 128) beside them."""
    for m, k, n in ((1, 1536, 1536), (16, 1536, 1536), (17, 5120, 640), (100, 640, 5120), (127, 1536, 256), (60, 1536, 120), (3, 200, 128)):
        x, w, b = O.make_inputs(m, k, n, seed=m + n)
        q = _quantised(k, n, w, b, fp8)
        y = q(x.to("cuda").view(1, m, k))
        assert y.shape == (1, m, n) and y.is_contiguous()
        y = y.view(m, n)
        if fp8:
            qw, sw = O.weight_quant_e4m3(w)
            ref = O.linear_e4m3(x, qw, sw, b)["out"]
            assert rel_l2(y, ref) < 2e-2
        else:
            qw, sw = O.weight_quant_int8(w)
            ref = O.linear_int8(x, qw, sw, b, keep_acc=False)["out"]
            np.testing.assert_array_equal(bf16_bits(y), bf16_bits(ref))
        poisoned = x.clone()                      # a NaN row stays a NaN row and stays alone, also in the padded buffer
        poisoned[m // 2, 5] = float("nan")
        yp = q(poisoned.to("cuda"))
        assert bool(torch.isnan(yp[m // 2]).all()) and bool(torch.equal(torch.isnan(yp).any(1).cpu(), torch.arange(m) == m // 2))


def test_q_k_v_separate_equals_n_concatenated():
    # the reference keeps to_q / to_k / to_v as three modules; one GEMM against the N-concatenated
    # weight is the benchmark's "fused QKV" shape.  Per-token / per-channel scales make them identical.
    m, k, n = 1000, 1536, 1536
    x, _, _ = O.make_inputs(m, k, 8, seed=7)
    ws, bs, outs = [], [], []
    for i in range(3):
        _, w, b = O.make_inputs(8, k, n, seed=10 + i)
        ws.append(w)
        bs.append(b)
        outs.append(_quantised(k, n, w, b, False)(x.to("cuda")))
    fused = _quantised(k, 3 * n, torch.cat(ws), torch.cat(bs), False)(x.to("cuda"))
    assert torch.equal(fused, torch.cat(outs, dim=1))
