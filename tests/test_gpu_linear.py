"""GPU parity of the MFMA GEMM + epilogue and of the swapped module against the oracle.

INT8: quantised activations, int32 accumulators and bf16 outputs are compared bit for bit.
FP8 : quantised activations bit for bit; outputs within 2e-2 relative L2 (the bound the task
      states; the reference's own accumulation order is unspecified), and in practice ~1e-3.
"""
import numpy as np
import pytest
import torch
from torch import nn

from oracle import daxq_oracle as O
from tests.util import bf16_bits, rel_l2

pytestmark = pytest.mark.gpu

VARIANTS = [0, 2, 5, 8, 11, 14]  # 0 = library default, 2 / 5 = generic kernel on 256x256 / 128x128 tiles, 8 / 11 / 14 = tiled kernel on 256x256 / 128x128 / 256x128 tiles


def _skip_if_too_small(variant, m, n):
    if variant in (8, 14) and (m < 256 or n < 256):
        pytest.skip("the 256x256 and 256x128 kernels need m, n >= 256")
    if variant == 11 and (m < 128 or n < 128):
        pytest.skip("the 128x128 kernel needs m, n >= 128")
FP8_TOL = 2e-2


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import dax_amd.ops as ops

    return ops


@pytest.fixture(autouse=True)
def _default_variant():
    yield
    from dax_amd import _capi

    _capi.debug_select_gemm(0)
    _capi.debug_select_gemm(2000)
    _capi.debug_select_gemm(3000)


def dev(t):
    return t.to("cuda") if t is not None else None


GEMM_SHAPES = [(256, 256, 128), (300, 520, 256), (1, 8, 128), (17, 24, 384), (512, 1536, 1536), (1000, 72, 640),
               (257, 257, 128), (4096, 1536, 1536), (200, 392, 384)]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_linear_i8_bit_exact(ops, variant, m, n, k):
    from dax_amd import _capi

    _skip_if_too_small(variant, m, n)
    _capi.debug_select_gemm(variant)
    x, w, b = O.make_inputs(m, k, n, seed=m + n + k)
    qw, sw = O.weight_quant_int8(w)
    ref = O.linear_int8(x, qw, sw, b)
    xq, sx = ops.act_quant_i8(dev(x))
    out, acc = ops.linear_i8_acc(xq, sx, dev(qw), dev(sw.view(-1)), dev(b))
    torch.cuda.synchronize()
    assert torch.equal(xq[:, :k].cpu(), ref["xq"])
    assert torch.equal(acc.cpu(), ref["acc"]), f"{(acc.cpu() != ref['acc']).sum().item()} accumulator mismatches"
    np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref["out"]))
    out2 = ops.linear_i8(xq, sx, dev(qw), dev(sw.view(-1)), None)
    ref2 = O.epilogue_int8(ref["acc"], ref["sx"], sw, None)
    np.testing.assert_array_equal(bf16_bits(out2), bf16_bits(ref2))


# tile grids (in 256-tiles) whose remainder band is 0 to 7 columns wide, with and without a partial last patch; the last
# two: tile rows under the last whole step of 8 (dense patches of 5 x 6 and 4 x 8 tiles) below whole patches
PATCH_SHAPES = [(256, 2048, 128), (1100, 2304, 128), (2600, 1024 + 256 * 2, 256), (700, 2048 + 256 * 3, 128), (2100, 256 * 4, 128),
                (1300, 2048 + 256 * 5, 128), (1500, 256 * 6, 256), (520, 4096 + 256 * 7, 128), (8500, 304, 128), (300, 5120, 384),
                (9100, 256 * 7, 128), (9450, 5120, 128), (3000, 256 * 7, 128)]


@pytest.mark.parametrize("order", [2002])
@pytest.mark.parametrize("m,n,k", PATCH_SHAPES)
def test_patch_tile_order_bit_exact(ops, m, n, k, order):
    """The 256x256 kernels in the banded tile order, which deals whole 32-slot patches to the XCDs (padding workgroups
    exit): every output tile is computed exactly once, accumulators and outputs equal the integer oracle's; FP8 equals
    the row-group order's bits."""
    from dax_amd import _capi

    _capi.debug_select_gemm(8)
    _capi.debug_select_gemm(order)
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, generator=g)
    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g)
    sx, sw = torch.rand(m, generator=g) + 0.5, torch.rand(n, generator=g) * 0.01
    b = torch.randn(n, generator=g).bfloat16()
    ref_acc = O.int_mm(xq, wq)
    ref_out = O.epilogue_int8(ref_acc, sx.view(-1, 1), sw.view(1, -1), b)
    out, acc = ops.linear_i8_acc(dev(xq), dev(sx), dev(wq), dev(sw), dev(b))
    assert torch.equal(acc.cpu(), ref_acc)
    np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref_out))
    out_plain = ops.linear_i8(dev(xq), dev(sx), dev(wq), dev(sw), dev(b))      # the launch without the accumulator dump
    np.testing.assert_array_equal(bf16_bits(out_plain), bf16_bits(ref_out))
    xf = torch.where((xq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), xq.view(torch.uint8))
    wf = torch.where((wq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), wq.view(torch.uint8))
    f_patch = ops.linear_e4m3(dev(xf), dev(sx), dev(wf), dev(sw), dev(b))
    _capi.debug_select_gemm(2001)
    f_rows = ops.linear_e4m3(dev(xf), dev(sx), dev(wf), dev(sw), dev(b))
    assert torch.equal(f_patch.view(torch.int16), f_rows.view(torch.int16))


# (m, n, k): grids of 256-tiles with one to four whole rounds of 256 workgroups and 1 to 64 tiles left over, edge tiles
# (shifted inwards) among the tiles left over
TAIL_SHAPES = [(4100, 4352, 128), (8500, 4096, 256), (4725, 13824, 128), (16300, 1024 + 40, 128), (8200, 8192 - 8, 128)]
# one to four whole rounds and between a quarter and a half of the CUs' worth of tiles left over (they run as halves of
# 256 x 128): K of one, two, three and many pairs of slices, edge tiles among the tiles left over
HALF_TAIL_SHAPES = [(4725, 5120, 128), (4725, 15360 - 24, 256), (9000, 2560, 384), (4725 - 3, 5120, 1152)]


# 256-tile rows of a grid of 20 tile columns, one per way the library cuts a launch by its tile count on 256 CUs: 60 tiles
# (128x128 tiles), 80 and 120 (every tile as two halves), 140 (whole tiles, part of a round), 260 and 320 (a round, the
# rest as quadrants), 340 and 380 (the rest as halves), 400 (two rounds of whole tiles)
CUT_ROWS = [3, 4, 6, 7, 13, 16, 17, 19, 20]


@pytest.mark.parametrize("tile_rows", CUT_ROWS)
def test_every_cut_of_a_launch_by_tile_count(ops, tile_rows):
    """The library's own choice (kernel argument 0) on either side of every tile count at which it changes the way a
    launch is cut into workgroups, ragged in both dimensions, K = 2048.  INT8: sampled rows (both edges of every tile
    row among them) against the integer oracle, and the whole output against the launch forced onto whole 256x256 tiles.
    FP8: the whole output is the bits of the launch forced onto whole 256x256 tiles."""
    from dax_amd import _capi

    m, n, k = 256 * tile_rows - 37, 5120 - 8, 2048
    g = torch.Generator().manual_seed(tile_rows)
    xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, generator=g)
    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g)
    sx = torch.rand(m, generator=g) * 0.02 + 1e-3
    sw = torch.rand(n, generator=g) * 0.002 + 1e-4
    b = (torch.randn(n, generator=g) * 0.5).bfloat16()
    xd, wd, sxd, swd, bd = dev(xq), dev(wq), dev(sx), dev(sw), dev(b)
    out = ops.linear_i8(xd, sxd, wd, swd, bd)
    edges = [r for t in range(tile_rows) for r in (256 * t, 256 * t + 255) if r < m] + [m - 256, m - 1]
    rows = torch.tensor(sorted(set(edges)) + torch.randint(0, m, (64,), generator=g).tolist())
    want = O.epilogue_int8(O.int_mm(xq[rows], wq), sx[rows].view(-1, 1), sw.view(1, -1), b)
    np.testing.assert_array_equal(bf16_bits(out[rows.to("cuda")]), bf16_bits(want))
    # any finite e4m3fn bytes
    x8 = torch.where((xq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), xq.view(torch.uint8)).cuda()
    w8 = torch.where((wq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), wq.view(torch.uint8)).cuda()
    swf = swd * 1e-3
    out8 = ops.linear_e4m3(x8, sxd, w8, swf, bd)
    _capi.debug_select_gemm(8)
    _capi.debug_select_gemm(3001)
    assert torch.equal(out.view(torch.int16), ops.linear_i8(xd, sxd, wd, swd, bd).view(torch.int16))
    whole8 = ops.linear_e4m3(x8, sxd, w8, swf, bd)
    assert bool(torch.isfinite(whole8.float()).all())
    assert torch.equal(out8.view(torch.int16), whole8.view(torch.int16)), "FP8 bits depend on how the launch is cut"


@pytest.mark.parametrize("m,n,k", TAIL_SHAPES + HALF_TAIL_SHAPES)
def test_last_round_in_smaller_pieces_bit_exact(ops, m, n, k):
    """A launch of 256x256 tiles whose last round of workgroups is a few tiles: the whole rounds run as 256x256 tiles,
    the tiles left over, in the workgroups behind them in the same grid, as their 128x128 quadrants or, with more than a
    quarter of the CUs' worth of them, as their 256x128 halves.  Accumulators and outputs equal the integer
    oracle's with the cut forced and by shape; FP8 outputs are the bits of the launch of whole tiles (every tile size
    runs the same sequence of MFMAs per output element)."""
    from dax_amd import _capi

    tiles = -(-m // 256) * -(-n // 256)
    if (m, n, k) in HALF_TAIL_SHAPES:
        assert tiles // 256 >= 1 and 64 < tiles % 256 <= 128, "the shape must leave a quarter to a half of 256 CUs' worth of tiles"
    else:
        assert tiles // 256 >= 1 and 0 < tiles % 256 <= 64, "the shape must leave at most a quarter of 256 CUs' worth of tiles"
    g = torch.Generator().manual_seed(m + n + k)
    xq = torch.randint(-127, 128, (m, k), dtype=torch.int8, generator=g)
    wq = torch.randint(-127, 128, (n, k), dtype=torch.int8, generator=g)
    sx, sw = torch.rand(m, generator=g) + 0.5, torch.rand(n, generator=g) * 0.01
    b = torch.randn(n, generator=g).bfloat16()
    ref_acc = O.int_mm(xq, wq)
    ref_out = O.epilogue_int8(ref_acc, sx.view(-1, 1), sw.view(1, -1), b)
    xf = torch.where((xq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), xq.view(torch.uint8))
    wf = torch.where((wq.view(torch.uint8) & 0x7f) == 0x7f, torch.zeros((), dtype=torch.uint8), wq.view(torch.uint8))
    _capi.debug_select_gemm(8)
    _capi.debug_select_gemm(2001)     # row groups: the order the cut exists for
    f8 = {}
    for tail in (3002, 3000, 3001):
        _capi.debug_select_gemm(tail)
        out, acc = ops.linear_i8_acc(dev(xq), dev(sx), dev(wq), dev(sw), dev(b))
        assert torch.equal(acc.cpu(), ref_acc), f"accumulators, tail choice {tail}"
        np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref_out))
        out_plain = ops.linear_i8(dev(xq), dev(sx), dev(wq), dev(sw), None)
        np.testing.assert_array_equal(bf16_bits(out_plain), bf16_bits(O.epilogue_int8(ref_acc, sx.view(-1, 1), sw.view(1, -1), None)))
        f8[tail] = ops.linear_e4m3(dev(xf), dev(sx), dev(wf), dev(sw), dev(b)).float().cpu()
    assert not torch.isnan(f8[3002]).any()
    assert torch.equal(f8[3002], f8[3001]), "FP8: the cut launch and the single launch must give the same bits"
    assert torch.equal(f8[3002], f8[3000]), "one to four whole rounds: the cut is taken by shape"


def test_tail_choice_bits_are_validated(ops):
    from dax_amd import _capi

    x = torch.zeros(256, 128, dtype=torch.int8, device="cuda")
    s = torch.ones(256, device="cuda")
    out = torch.empty(256, 256, dtype=torch.bfloat16, device="cuda")
    rc = _capi.lib().daxq_linear_w8a8(0, 0, 0, x.data_ptr(), 128, s.data_ptr(), x.data_ptr(), 128, s.data_ptr(), None, out.data_ptr(), 256,
                                      None, 0, 256, 256, 128, 3 << 28, torch.cuda.current_stream().cuda_stream)
    assert rc < 0 and "tail" in _capi.last_error()


def _random_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        m = int(rng.integers(256, 1400))
        n = int(rng.integers(32, 160)) * 8           # any multiple of 8 from 256 up
        k = int(rng.integers(1, 13)) * 128
        shapes.append((m, n, k, int(rng.integers(0, 3)) * 128, int(rng.integers(0, 5)) * 8))
    return shapes


@pytest.mark.parametrize("variant", [8, 11, 14, 2, 8 | (2 << 24), 8 | (1 << 24)])
@pytest.mark.parametrize("m,n,k,pad_k,pad_n", _random_shapes(14, seed=2024))
def test_linear_i8_random_shapes_and_strides_bit_exact(ops, variant, m, n, k, pad_k, pad_n):
    """Seeded random M, N, K (edge tiles shifted inwards in both directions, short and long K) with padded leading
    dimensions, raw int8 operands straight through the C ABI: accumulators and outputs against the integer oracle.
    (Bits 24-27 of the kernel argument: the banded order and the row groups on the same operands.)"""
    from dax_amd import _capi

    _capi.debug_select_gemm(variant & 0xffff)
    g = torch.Generator("cpu").manual_seed(m * 7 + n * 3 + k)
    xq = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
    wq = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
    sx = (torch.rand(m, generator=g) * 0.02 + 1e-3).float()
    sw = (torch.rand(n, generator=g) * 0.002 + 1e-4).float()
    b = (torch.randn(n, generator=g) * 0.5).bfloat16()
    want_acc = O.int_mm(xq, wq)
    want_out = O.epilogue_int8(want_acc, sx.view(-1, 1), sw.view(1, -1), b)
    xq_wide = torch.full((m, k + pad_k), 5, dtype=torch.int8, device="cuda")
    xq_wide[:, :k] = dev(xq)
    wq_wide = torch.full((n, k + pad_k), -7, dtype=torch.int8, device="cuda")
    wq_wide[:, :k] = dev(wq)
    out_wide = torch.full((m, n + pad_n), 3.0, dtype=torch.bfloat16, device="cuda")
    acc_wide = torch.full((m, n + pad_n), -1, dtype=torch.int32, device="cuda")
    sxd, swd, bd = dev(sx), dev(sw), dev(b)
    # the general entry point names its kernel per call (the library keeps no selection of its own)
    rc = _capi.lib().daxq_linear_w8a8(0, 0, 0, xq_wide.data_ptr(), k + pad_k, sxd.data_ptr(), wq_wide.data_ptr(), k + pad_k,
                                      swd.data_ptr(), bd.data_ptr(), out_wide.data_ptr(), n + pad_n, acc_wide.data_ptr(),
                                      n + pad_n, m, n, k, variant, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "linear_i8")
    torch.cuda.synchronize()
    assert torch.equal(acc_wide[:, :n].cpu(), want_acc)
    np.testing.assert_array_equal(bf16_bits(out_wide[:, :n]), bf16_bits(want_out))
    assert bool((out_wide[:, n:] == 3.0).all()) and bool((acc_wide[:, n:] == -1).all())   # nothing outside


@pytest.mark.parametrize("variant", VARIANTS)
def test_linear_i8_adversarial_extremes(ops, variant):
    from dax_amd import _capi

    _capi.debug_select_gemm(variant)
    m, n, k = 300, 264, 13824
    xq = torch.full((m, k), -128, dtype=torch.int8)
    xq[1::2] = 127
    wq = torch.full((n, k), -128, dtype=torch.int8)
    wq[::3] = 127
    wq[5, ::2] = 1
    sx = torch.full((m,), 2.0 ** -10)
    sw = torch.full((n,), 2.0 ** -12)
    out, acc = ops.linear_i8_acc(dev(xq), dev(sx), dev(wq), dev(sw), None)
    want = O.int_mm(xq, wq)
    assert torch.equal(acc.cpu(), want)
    assert int(want.max()) == 128 * 128 * k
    np.testing.assert_array_equal(bf16_bits(out), bf16_bits(O.epilogue_int8(want, sx.view(-1, 1), sw.view(1, -1), None)))


@pytest.mark.parametrize("variant", [0, 2, 8, 11, 14])
def test_linear_i8_one_hot_layout(ops, variant):
    # a single non-zero in each operand lands in exactly one accumulator: catches any
    # row/column or operand transposition inside the MFMA tiling
    from dax_amd import _capi

    _capi.debug_select_gemm(variant)
    m, n, k = 300, 300, 256
    rng = np.random.default_rng(0)
    for _ in range(6):
        i, j, kk = int(rng.integers(m)), int(rng.integers(n)), int(rng.integers(k))
        xq = torch.zeros(m, k, dtype=torch.int8)
        wq = torch.zeros(n, k, dtype=torch.int8)
        xq[i, kk] = 3
        wq[j, kk] = -5
        _, acc = ops.linear_i8_acc(dev(xq), dev(torch.ones(m)), dev(wq), dev(torch.ones(n)), None)
        acc = acc.cpu()
        assert acc[i, j] == -15 and acc.abs().sum() == 15, (i, j, kk)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (300, 520, 256), (17, 24, 384), (512, 1536, 1536)])
def test_linear_e4m3_within_tolerance(ops, variant, m, n, k):
    from dax_amd import _capi

    _skip_if_too_small(variant, m, n)
    _capi.debug_select_gemm(variant)
    x, w, b = O.make_inputs(m, k, n, seed=m + n + k + 1)
    qw, sw = O.weight_quant_e4m3(w)
    ref = O.linear_e4m3(x, qw, sw, b)
    xq, sx = ops.act_quant_e4m3(dev(x))
    assert torch.equal(xq[:, :k].cpu(), ref["xq"].view(torch.uint8))
    out, acc = ops.linear_e4m3_acc(xq, sx, dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b))
    acc_ref = ref["xq"].float() @ qw.float().t()
    # fp32 accumulators; the fp8 MFMA sums the 64 products of one instruction in a common-exponent
    # adder of limited width, so it deviates from an fp32 sum at the 1e-5 level (measured <= 4e-5)
    assert rel_l2(acc, acc_ref) < 2e-4
    r = rel_l2(out, ref["out"])
    assert r < FP8_TOL, r
    assert r < 3e-3, r                          # what fp32 accumulation actually delivers


@pytest.mark.parametrize("variant", [8, 11, 14, 2])
@pytest.mark.parametrize("e5m2", [False, True])
@pytest.mark.parametrize("m,n,k,pad_k,pad_n", _random_shapes(8, seed=77))
def test_linear_fp8_random_shapes_accumulators(ops, variant, e5m2, m, n, k, pad_k, pad_n):
    """Seeded random shapes with padded leading dimensions and raw fp8 bytes through the C ABI: the fp32 accumulators
    against the exact sum of the decoded products (float64), element by element."""
    from dax_amd import _capi

    _capi.debug_select_gemm(variant)
    g = torch.Generator("cpu").manual_seed(m + 5 * n + 11 * k)
    act_dtype = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    xf = (torch.randn(m, k, generator=g) * 3).to(act_dtype)
    wf = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    want = xf.double() @ wf.double().t()
    bound = xf.double().abs() @ wf.double().abs().t()          # sum of |products|: the scale of the rounding error
    xq_wide = torch.zeros((m, k + pad_k), dtype=torch.uint8, device="cuda")
    xq_wide[:, :k] = dev(xf.view(torch.uint8))
    wq_wide = torch.zeros((n, k + pad_k), dtype=torch.uint8, device="cuda")
    wq_wide[:, :k] = dev(wf.view(torch.uint8))
    out_wide = torch.zeros((m, n + pad_n), dtype=torch.bfloat16, device="cuda")
    acc_wide = torch.full((m, n + pad_n), -1.0, dtype=torch.float32, device="cuda")
    ones_m, ones_n = torch.ones(m, device="cuda"), torch.ones(n, device="cuda")
    if variant == 0:   # the named entry points (library's own choice of kernel)
        fn = _capi.lib().daxq_linear_e5m2_e4m3 if e5m2 else _capi.lib().daxq_linear_e4m3
        rc = fn(xq_wide.data_ptr(), k + pad_k, ones_m.data_ptr(), wq_wide.data_ptr(), k + pad_k, ones_n.data_ptr(), None,
                out_wide.data_ptr(), n + pad_n, acc_wide.data_ptr(), n + pad_n, m, n, k,
                torch.cuda.current_stream().cuda_stream)
    else:
        rc = _capi.lib().daxq_linear_w8a8(2 if e5m2 else 1, 1, 0, xq_wide.data_ptr(), k + pad_k, ones_m.data_ptr(),
                                          wq_wide.data_ptr(), k + pad_k, ones_n.data_ptr(), None, out_wide.data_ptr(),
                                          n + pad_n, acc_wide.data_ptr(), n + pad_n, m, n, k, variant,
                                          torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "linear fp8")
    torch.cuda.synchronize()
    got = acc_wide[:, :n].cpu().double()
    err = ((got - want).abs() / bound.clamp_min(1e-30)).max().item()
    assert err < 2e-5, err        # fp32 accumulation of K products: a few 2^-24 of the sum of magnitudes
    assert bool((acc_wide[:, n:] == -1.0).all())
    assert torch.equal(out_wide[:, :n].cpu(), acc_wide[:, :n].cpu().bfloat16())   # unit scales, no bias: out = bf16(acc)


@pytest.mark.parametrize("variant", [8, 11, 14])
@pytest.mark.parametrize("k", [128, 256, 384, 512, 640, 768, 896, 1024, 1152, 1280, 1408, 1536])
def test_fp8_16x16x128_form_every_count_of_slice_pairs(ops, k, variant):
    """Every number of 128-byte pairs of K slices from 1 to 12 on the three tile sizes: the plain loop below four pairs,
    then first pair, steady pairs in twos, the odd one and the register moves in front of the three tail pairs all occur.
    Accumulators against exact float64 sums, element by element, on a grid of tiles with ragged edges; every tile size
    gives the same bits."""
    from dax_amd import _capi

    m, n = 300, 700
    g = torch.Generator("cpu").manual_seed(k)
    xf = (torch.randn(m, k, generator=g) * 3).to(torch.float8_e4m3fn)
    wf = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    want = xf.double() @ wf.double().t()
    bound = xf.double().abs() @ wf.double().abs().t()
    _capi.debug_select_gemm(variant)
    sx, sw = torch.rand(m, generator=g) + 0.5, torch.rand(n, generator=g) + 0.5
    b = torch.randn(n, generator=g).bfloat16()
    out, acc = ops.linear_e4m3_acc(dev(xf.view(torch.uint8)), dev(sx), dev(wf.view(torch.uint8)), dev(sw), dev(b))
    err = ((acc.cpu().double() - want).abs() / bound.clamp_min(1e-30)).max().item()
    # (the MFMA adds the 128 products of an instruction in a fixed-point adder of limited width: with one to three
    # instructions per sum that error, about 3e-5 of the sum of magnitudes, is not averaged down yet)
    assert err < (4e-5 if k < 512 else 2e-5), err
    ref = (acc.cpu() * sx.view(-1, 1) * sw.view(1, -1) + b.float()).bfloat16()     # the epilogue on the kernel's own sums
    np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref))
    _capi.debug_select_gemm(8 if variant == 11 else 11)
    out2, acc2 = ops.linear_e4m3_acc(dev(xf.view(torch.uint8)), dev(sx), dev(wf.view(torch.uint8)), dev(sw), dev(b))
    assert torch.equal(acc, acc2) and torch.equal(out, out2), "every tile size must give the same FP8 bits"


@pytest.mark.parametrize("k", [3968, 4096, 4224, 4352, 4480, 5120, 13824])
def test_nine_stage_128_tile_form_every_count_of_slice_pairs(ops, k):
    """Launches of at most 256 tiles of 128x128 with K >= 4096 run the five-stage pipeline with nine stages (four pairs
    of slices in flight): the shortest K it takes, odd and even pair counts, one K below it (the five-stage form), and
    the depths of the cross-attention and FFN-down projections.  INT8 accumulators and outputs against the integer oracle, FP8 accumulators
    against exact float64 sums, on a 3 x 6 grid of tiles with ragged edges, chosen by shape and by argument."""
    from dax_amd import _capi

    m, n = 300, 700
    g = torch.Generator("cpu").manual_seed(k)
    xq = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int32).to(torch.int8)
    wq = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int32).to(torch.int8)
    sx, sw = torch.rand(m, generator=g) * 0.02 + 1e-3, torch.rand(n, generator=g) * 0.002 + 1e-4
    b = torch.randn(n, generator=g).bfloat16()
    want_acc = O.int_mm(xq, wq)
    want_out = O.epilogue_int8(want_acc, sx.view(-1, 1), sw.view(1, -1), b)
    xf = (torch.randn(m, k, generator=g) * 3).to(torch.float8_e4m3fn)
    wf = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    want_f = xf.double() @ wf.double().t()
    bound = xf.double().abs() @ wf.double().abs().t()
    for variant in (11, 0):     # 300 x 700 has 6 tiles of 256x256: the library's own choice is the 128-tile form too
        _capi.debug_select_gemm(variant)
        out, acc = ops.linear_i8_acc(dev(xq), dev(sx), dev(wq), dev(sw), dev(b))
        assert torch.equal(acc.cpu(), want_acc)
        np.testing.assert_array_equal(bf16_bits(out), bf16_bits(want_out))
        np.testing.assert_array_equal(bf16_bits(ops.linear_i8(dev(xq), dev(sx), dev(wq), dev(sw), dev(b))), bf16_bits(want_out))
        outf, accf = ops.linear_e4m3_acc(dev(xf.view(torch.uint8)), dev(sx), dev(wf.view(torch.uint8)), dev(sw), dev(b))
        err = ((accf.cpu().double() - want_f).abs() / bound.clamp_min(1e-30)).max().item()
        assert err < 2e-5, err
        ref = (accf.cpu() * sx.view(-1, 1) * sw.view(1, -1) + b.float()).bfloat16()
        np.testing.assert_array_equal(bf16_bits(outf), bf16_bits(ref))


@pytest.mark.parametrize("e5m2", [False, True])
@pytest.mark.parametrize("m,n,k", [(8192, 5120, 5120), (4096, 5120, 13824), (2304, 2560, 640)])
def test_fp8_16x16x128_form_against_the_32x32x64_form_every_element(ops, m, n, k, e5m2):
    """The FP8 kernel on 16x16x128 MFMAs (fragments refilled in place behind the MFMAs that read them) against the
    generic kernel (32x32x64 MFMAs) at full depth of K and with every CU busy: raw fp32 accumulators of the whole
    output, element by element, within the rounding of an fp32 sum (a wrong or torn operand would be off by orders of
    magnitude); three launches, identical bits each time, and the 128x128-tile launch the same bits again; a row sample
    against the exact float64 sum."""
    from dax_amd import _capi

    g = torch.Generator("cpu").manual_seed(m + n + k)
    act_dtype = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    xf = (torch.randn(m, k, generator=g) * 3).to(act_dtype)
    wf = (torch.randn(n, k, generator=g) * 0.5).to(torch.float8_e4m3fn)
    xd, wd = dev(xf.view(torch.uint8)), dev(wf.view(torch.uint8))
    one_m, one_n = torch.ones(m, device="cuda"), torch.ones(n, device="cuda")
    fn = ops.linear_e5m2_e4m3_acc if e5m2 else ops.linear_e4m3_acc
    _capi.debug_select_gemm(2)
    _, acc_wide = fn(xd, one_m, wd, one_n, None)
    _capi.debug_select_gemm(8)
    runs = [fn(xd, one_m, wd, one_n, None)[1] for _ in range(3)]
    assert torch.equal(runs[0], runs[1]) and torch.equal(runs[0], runs[2])
    _capi.debug_select_gemm(11)
    assert torch.equal(runs[0], fn(xd, one_m, wd, one_n, None)[1]), "128x128 tiles: the same sums"
    bound = dev(xf.float().abs()) @ dev(wf.float().abs()).t()      # sum of |products| (fp32 on the device is enough for a bound)
    err = ((runs[0] - acc_wide).abs() / bound.clamp_min(1e-30)).max().item()
    assert err < 4e-5, err
    rows = torch.randint(0, m, (48,), generator=g)
    want = xf[rows].double() @ wf.double().t()
    b64 = xf[rows].double().abs() @ wf.double().abs().t()
    err = ((runs[0][dev(rows)].cpu().double() - want).abs() / b64.clamp_min(1e-30)).max().item()
    assert err < 2e-5, err


@pytest.mark.parametrize("variant", [0, 5, 8])
@pytest.mark.parametrize("m,n,k", [(300, 520, 256), (17, 24, 384), (512, 1536, 1536), (4096, 1536, 1536)])
def test_linear_e5m2_activations_within_tolerance(ops, variant, m, n, k):
    from dax_amd import _capi

    _skip_if_too_small(variant, m, n)
    _capi.debug_select_gemm(variant)
    x, w, b = O.make_inputs(m, k, n, seed=m + n + k + 2)
    qw, sw = O.weight_quant_e4m3(w)
    ref = O.linear_e4m3(x, qw, sw, b, act_dtype=torch.float8_e5m2)
    xq, sx = ops.act_quant_e5m2(dev(x))
    assert torch.equal(xq[:, :k].cpu(), ref["xq"].view(torch.uint8))
    out, acc = ops.linear_e5m2_e4m3_acc(xq, sx, dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b))
    acc_ref = ref["xq"].float() @ qw.float().t()
    assert rel_l2(acc, acc_ref) < 2e-4          # a wrong operand format would be off by orders of magnitude
    assert rel_l2(out, ref["out"]) < 3e-3


def test_linear_rejects_unaligned_k(ops):
    from dax_amd._capi import DaxqError

    xq = torch.zeros(8, 64, dtype=torch.int8, device="cuda")
    wq = torch.zeros(8, 64, dtype=torch.int8, device="cuda")
    with pytest.raises(DaxqError, match="multiple of 128"):
        ops.linear_i8(xq, torch.ones(8, device="cuda"), wq, torch.ones(8, device="cuda"), None)


@pytest.mark.parametrize("variant", [0, 5, 2, 8, 11, 14])
def test_linear_leading_dimensions_through_the_c_abi(ops, variant):
    """Operands and output as column slices of wider buffers (ld > logical width), straight through the C ABI:
    what a caller does that writes q | k | v into one [M, 3N] tensor with three launches."""
    from dax_amd import _capi

    _capi.debug_select_gemm(variant)
    m, n, k = 600, 520, 384
    x, w, b = O.make_inputs(m, k, n, seed=77)
    qw, sw = O.weight_quant_int8(w)
    ref = O.linear_int8(x, qw, sw, b)
    xq_wide = torch.full((m, k + 128), 7, dtype=torch.int8, device="cuda")
    xq_wide[:, :k] = dev(ref["xq"])
    wq_wide = torch.full((n, k + 256), -3, dtype=torch.int8, device="cuda")
    wq_wide[:, :k] = dev(qw)
    out_wide = torch.full((m, 3 * n + 8), 1.0, dtype=torch.bfloat16, device="cuda")
    acc_wide = torch.zeros((m, n + 4), dtype=torch.int32, device="cuda")
    sx, swd, bd = dev(ref["sx"].reshape(-1).contiguous()), dev(sw.reshape(-1).contiguous()), dev(b)
    col0 = n + 8                                                    # 16-byte aligned column offset
    if variant == 0:
        rc = _capi.lib().daxq_linear_i8(xq_wide.data_ptr(), k + 128, sx.data_ptr(), wq_wide.data_ptr(), k + 256, swd.data_ptr(),
                                        bd.data_ptr(), out_wide.data_ptr() + 2 * col0, 3 * n + 8, acc_wide.data_ptr(), n + 4,
                                        m, n, k, torch.cuda.current_stream().cuda_stream)
    else:
        rc = _capi.lib().daxq_linear_w8a8(0, 0, 0, xq_wide.data_ptr(), k + 128, sx.data_ptr(), wq_wide.data_ptr(), k + 256,
                                          swd.data_ptr(), bd.data_ptr(), out_wide.data_ptr() + 2 * col0, 3 * n + 8,
                                          acc_wide.data_ptr(), n + 4, m, n, k, variant, torch.cuda.current_stream().cuda_stream)
    _capi.check(rc, "linear_i8")
    torch.cuda.synchronize()
    assert torch.equal(out_wide[:, col0:col0 + n].cpu().view(torch.int16), ref["out"].view(torch.int16))
    assert torch.equal(acc_wide[:, :n].cpu(), ref["acc"])
    assert bool((out_wide[:, :col0] == 1).all()) and bool((out_wide[:, col0 + n:] == 1).all())   # nothing outside the slice
    assert bool((acc_wide[:, n:] == 0).all())
    _capi.debug_select_gemm(0)


# --------------------------------------------------------------------------- the swapped module
class ToyBlock(nn.Module):
    def __init__(self, d=256, f=520):
        super().__init__()
        self.to_q = nn.Linear(d, d)
        self.ffn = nn.Sequential(nn.Linear(d, f), nn.GELU(approximate="tanh"), nn.Linear(f, d, bias=False))
        self.proj_out = nn.Linear(d, 64)

    def forward(self, x):
        return self.proj_out(self.ffn(self.to_q(x)))


def _toy(seed=0):
    torch.manual_seed(seed)
    m = ToyBlock().bfloat16()
    with torch.no_grad():
        for p in m.parameters():
            p.mul_(0.5)
    return m


@pytest.mark.parametrize("home", ["cuda", "cpu"])
def test_quantize_dynamic_int8_module_matches_oracle(home):
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    model = _toy().to(home)
    w = model.to_q.weight.detach().cpu().clone()
    b = model.to_q.bias.detach().cpu().clone()
    quantize_dynamic(model, {"": cfg(), "proj_out": None})
    assert isinstance(model.to_q, QLinear) and isinstance(model.ffn[0], QLinear) and isinstance(model.ffn[2], QLinear)
    assert type(model.proj_out) is nn.Linear
    assert model.to_q.qweight.device.type == home
    qw, sw = O.weight_quant_int8(w)
    assert torch.equal(model.to_q.qweight.cpu(), qw)
    assert torch.equal(model.to_q.weight_scale.cpu(), sw)
    assert model.to_q.weight_scale.shape == (1, 256) and model.to_q.weight_scale.dtype == torch.float32
    assert set(model.to_q.state_dict().keys()) == {"qweight", "weight_scale", "bias"}
    assert model.ffn[2].bias is None
    model = model.to("cuda")
    x, _, _ = O.make_inputs(2 * 75, 256, 8, seed=2)
    y = model.to_q(x.view(2, 75, 256).to("cuda"))
    assert y.shape == (2, 75, 256) and y.dtype == torch.bfloat16
    ref = O.linear_int8(x, qw, sw, b)["out"]
    np.testing.assert_array_equal(bf16_bits(y.view(-1, 256)), bf16_bits(ref))
    # dequantised weight property
    assert torch.equal(model.to_q.weight.cpu(), O.dequant_weight(qw, sw))
    # whole block runs (K=520 is not a multiple of 128: padded operands)
    z = model(x.view(2, 75, 256).to("cuda"))
    h = O.linear_int8(x, qw, sw, b)["out"]
    qw1, sw1 = model.ffn[0].qweight.cpu(), model.ffn[0].weight_scale.cpu()
    h = O.linear_int8(h, qw1, sw1, model.ffn[0].bias.detach().cpu())["out"]
    h = torch.nn.functional.gelu(h.to("cuda"), approximate="tanh").cpu()
    h = O.linear_int8(h, model.ffn[2].qweight.cpu(), model.ffn[2].weight_scale.cpu(), None)["out"]
    h = torch.nn.functional.linear(h.to("cuda"), model.proj_out.weight, model.proj_out.bias)
    np.testing.assert_array_equal(bf16_bits(z.view(-1, 64)), bf16_bits(h))


def test_module_takes_the_input_shapes_of_nn_linear():
    """[..., K] -> [..., N] for any leading shape the reference's view(-1, K) accepts (dynamic/linear.py:181-183,
    :224-226): no token at all, a single vector, several leading dimensions, a view with strided columns."""
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    model = _toy(4).to("cuda")
    w, b = model.to_q.weight.detach().cpu().clone(), model.to_q.bias.detach().cpu().clone()
    quantize_dynamic(model, {"": cfg(), "proj_out": None})
    qw, sw = O.weight_quant_int8(w)
    lin = model.to_q
    for shape in [(0, 256), (2, 0, 256), (256,), (1, 256), (2, 3, 5, 256)]:
        g = torch.Generator("cpu").manual_seed(len(shape))
        x = torch.randn(*shape, generator=g).bfloat16()
        y = lin(x.to("cuda"))
        assert y.shape == shape[:-1] + (256,) and y.dtype == torch.bfloat16
        if x.numel():
            ref = O.linear_int8(x.reshape(-1, 256), qw, sw, b)["out"]
            np.testing.assert_array_equal(bf16_bits(y.reshape(-1, 256)), bf16_bits(ref))
    wide = torch.randn(10, 512, generator=torch.Generator("cpu").manual_seed(9)).bfloat16()
    y = lin(wide.to("cuda")[:, ::2])                      # every second column: a view, not contiguous rows
    ref = O.linear_int8(wide[:, ::2].contiguous(), qw, sw, b)["out"]
    np.testing.assert_array_equal(bf16_bits(y), bf16_bits(ref))
    with pytest.raises(RuntimeError):                      # not flattenable by view: the reference raises as well
        lin(torch.randn(2, 5, 256, device="cuda").bfloat16().transpose(0, 1))


def test_quantize_dynamic_fp8_module_matches_oracle():
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_fp8_per_token_act_per_channel_weight_qconfig as cfg

    model = _toy(1).to("cuda")
    w = model.to_q.weight.detach().cpu().clone()
    b = model.to_q.bias.detach().cpu().clone()
    quantize_dynamic(model, {"": cfg(activation_dtype=torch.float8_e4m3fn), "proj_out": None})
    assert isinstance(model.to_q, QLinear) and model.to_q.compute_dtype == "FP8"
    assert model.to_q.qweight.dtype == torch.float8_e4m3fn
    qw, sw = O.weight_quant_e4m3(w)
    assert torch.equal(model.to_q.qweight.cpu().view(torch.uint8), qw.view(torch.uint8))
    assert torch.equal(model.to_q.weight_scale.cpu(), sw)
    x, _, _ = O.make_inputs(150, 256, 8, seed=3)
    y = model.to_q(x.to("cuda"))
    ref = O.linear_e4m3(x, qw, sw, b)["out"]
    assert rel_l2(y, ref) < FP8_TOL


def test_fp8_default_qconfig_e5m2_activations_e4m3_weights():
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_fp8_per_token_act_per_channel_weight_qconfig as cfg

    model = _toy(2).to("cuda")
    w = model.to_q.weight.detach().cpu().clone()
    b = model.to_q.bias.detach().cpu().clone()
    quantize_dynamic(model, {"": cfg(), "proj_out": None})       # the reference's default FP8 pairing
    assert isinstance(model.to_q, QLinear) and model.to_q.input_dtype == torch.float8_e5m2
    assert model.to_q.qweight.dtype == torch.float8_e4m3fn
    qw, sw = O.weight_quant_e4m3(w)
    x, _, _ = O.make_inputs(150, 256, 8, seed=5)
    y = model.to_q(x.to("cuda"))
    ref = O.linear_e4m3(x, qw, sw, b, act_dtype=torch.float8_e5m2)["out"]
    assert rel_l2(y, ref) < FP8_TOL
    # e5m2 weights (any of FP8_ALLOWED_DTYPES is a valid weight dtype, dax/quant/nn/dynamic/linear.py:42-43)
    model2 = _toy(3).to("cuda")
    w2 = model2.to_q.weight.detach().cpu().clone()
    b2 = model2.to_q.bias.detach().cpu().clone()
    quantize_dynamic(model2, {"": cfg(weight_dtype=torch.float8_e5m2)})
    assert isinstance(model2.to_q, QLinear) and model2.to_q.qweight.dtype == torch.float8_e5m2
    qw2, sw2 = O.weight_quant_fp8(w2, torch.float8_e5m2)
    assert torch.equal(model2.to_q.qweight.cpu().view(torch.uint8), qw2.view(torch.uint8))
    assert torch.equal(model2.to_q.weight_scale.cpu(), sw2)
    y2 = model2.to_q(x.to("cuda"))
    ref2 = O.linear_fp8(x, qw2, sw2, b2, act_dtype=torch.float8_e5m2)["out"]
    assert rel_l2(y2, ref2) < FP8_TOL


def test_state_dict_round_trip_and_hooks():
    from dax_amd.quant.nn.dynamic import Linear as QLinear
    from dax_amd.quant.qscheme import per_channel_symmetric, per_token_symmetric
    from dax_amd.quant.quantization import quantize_dynamic
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig as cfg

    model = _toy(3).to("cuda")
    calls = []
    model.to_q.register_forward_hook(lambda mod, inp, out: calls.append("post"))
    model.to_q.register_forward_pre_hook(lambda mod, inp: calls.append("pre"))
    quantize_dynamic(model, {"": cfg()})
    x = torch.randn(20, 256, device="cuda").bfloat16()
    y = model.to_q(x)
    assert calls == ["pre", "post"]
    fresh = QLinear(256, 256, True, None, torch.int8, torch.int8, torch.bfloat16, per_channel_symmetric,
                    per_token_symmetric)
    fresh.load_state_dict(model.to_q.state_dict())
    fresh = fresh.to("cuda")
    assert torch.equal(fresh(x), y)


# --------------------------------------------------------------------------- full-size properties
@pytest.mark.parametrize("fp8", [False, True])
def test_full_size_14b_out_proj_rows_and_checksum(ops, fp8):
    """M=75600, K=5120, N=5120 (Wan2.1-14B 720p out-projection).  Rows are independent, so a
    sample of rows (incl. the first / last rows of the first / last tiles) is checked against
    the oracle exactly; the whole accumulator matrix is checked through the identity
    sum_ij acc[i,j] = sum_k (sum_i xq[i,k]) * (sum_j wq[j,k])."""
    m, k, n = 75600, 5120, 5120
    x, w, b = O.make_inputs(m, k, n, seed=2)
    xd = dev(x)
    rows = torch.cat([torch.arange(0, 3), torch.arange(255, 258), torch.arange(m - 82, m - 78), torch.arange(m - 3, m),
                      torch.randint(0, m, (180,), generator=torch.Generator().manual_seed(0))]).unique()
    if fp8:
        qw, sw = O.weight_quant_e4m3(w)
        xq, sx = ops.act_quant_e4m3(xd)
        out, acc = ops.linear_e4m3_acc(xq, sx, dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b))
        ref = O.linear_e4m3(x[rows], qw, sw, b)
        assert torch.equal(xq[rows.to("cuda")][:, :k].cpu(), ref["xq"].view(torch.uint8))
        assert rel_l2(out[rows.to("cuda")], ref["out"]) < FP8_TOL
        # linearity of the fp32 accumulation in the row sums (tolerance: fp32 summation)
        tot = acc.double().sum().item()
        xs = xq[:, :k].view(torch.float8_e4m3fn).float().sum(0).double()
        ws = dev(qw).float().sum(0).double()
        want = float((xs * ws).sum().item())
        assert abs(tot - want) <= 1e-4 * max(1.0, abs(want))
    else:
        qw, sw = O.weight_quant_int8(w)
        xq, sx = ops.act_quant_i8(xd)
        out, acc = ops.linear_i8_acc(xq, sx, dev(qw), dev(sw.view(-1)), dev(b))
        ref = O.linear_int8(x[rows], qw, sw, b)
        rd = rows.to("cuda")
        assert torch.equal(xq[rd][:, :k].cpu(), ref["xq"])
        assert torch.equal(sx[rd].cpu(), ref["sx"].view(-1))
        assert torch.equal(acc[rd].cpu(), ref["acc"])
        np.testing.assert_array_equal(bf16_bits(out[rd]), bf16_bits(ref["out"]))
        tot = int(acc.sum(dtype=torch.int64).item())
        xs = xq[:, :k].sum(0, dtype=torch.int64)
        ws = dev(qw).sum(0, dtype=torch.int64)
        assert tot == int((xs * ws).sum().item())
        # idempotence: a second launch over the same operands gives the same bits
        out2 = ops.linear_i8(xq, sx, dev(qw), dev(sw.view(-1)), dev(b))
        assert torch.equal(out2, out)


# ------------------------------------------------------------------ split-K (few output tiles)
@pytest.mark.parametrize("m,n,k,splits", [(512, 5120, 5120, 2), (512, 5120, 5120, 4), (300, 520, 1024, 2), (128, 128, 1024, 8),
                                          (1000, 392, 1536, 3), (512, 5120, 5120, 0), (256, 5120, 5120, 0)])
def test_linear_i8_splitk_bit_exact(ops, m, n, k, splits):
    """K cut into ranges that run as separate workgroups: integer partial sums, so outputs equal the oracle's bit for bit;
    two calls in a row on the same workspace (the counters are left at zero), the second on another problem."""
    x, w, b = O.make_inputs(m, k, n, seed=m + n + k + splits)
    qw, sw = O.weight_quant_int8(w)
    ref = O.linear_int8(x, qw, sw, b)
    xq, sx = ops.act_quant_i8(dev(x))
    out = ops.linear_w8a8_splitk(xq, sx, dev(qw), dev(sw.view(-1)), dev(b), "i8", "i8", splits)
    np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref["out"]))
    out_nb = ops.linear_w8a8_splitk(xq[: m - 100 if m > 300 else m], sx[: m - 100 if m > 300 else m], dev(qw), dev(sw.view(-1)), None,
                                    "i8", "i8", splits)
    rows = m - 100 if m > 300 else m
    ref_nb = O.epilogue_int8(ref["acc"][:rows], ref["sx"][:rows], sw, None)
    np.testing.assert_array_equal(bf16_bits(out_nb), bf16_bits(ref_nb))
    out2 = ops.linear_w8a8_splitk(xq, sx, dev(qw), dev(sw.view(-1)), dev(b), "i8", "i8", splits)
    np.testing.assert_array_equal(bf16_bits(out2), bf16_bits(ref["out"]))


def test_splitk_workspace_shared_by_launches_of_different_shapes(ops):
    """One workspace, a launch with few tiles and many ranges, then one with more tiles: the second launch's counters
    must not sit where the first one kept partial results."""
    cases = [(172, 5120, 13824, 6), (512, 5120, 5120, 2), (300, 640, 1024, 4), (512, 5120, 5120, 2)]
    for m, n, k, splits in cases:
        x, w, b = O.make_inputs(m, k, n, seed=k + splits)
        qw, sw = O.weight_quant_int8(w)
        ref = O.linear_int8(x, qw, sw, b, keep_acc=False)["out"]
        xq, sx = ops.act_quant_i8(dev(x))
        out = ops.linear_w8a8_splitk(xq, sx, dev(qw), dev(sw.view(-1)), dev(b), "i8", "i8", splits)
        np.testing.assert_array_equal(bf16_bits(out), bf16_bits(ref), err_msg=str((m, n, k, splits)))


@pytest.mark.parametrize("e5m2", [False, True])
def test_linear_fp8_splitk_within_tolerance_and_deterministic(ops, e5m2):
    m, n, k = 512, 1536, 2048
    x, w, b = O.make_inputs(m, k, n, seed=91)
    qw, sw = O.weight_quant_e4m3(w)
    act = torch.float8_e5m2 if e5m2 else torch.float8_e4m3fn
    ref = O.linear_fp8(x, qw, sw, b, act_dtype=act)
    xq, sx = (ops.act_quant_e5m2 if e5m2 else ops.act_quant_e4m3)(dev(x))
    fmt = "e5m2" if e5m2 else "e4m3"
    outs = [ops.linear_w8a8_splitk(xq, sx, dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b), fmt, "e4m3", 4) for _ in range(3)]
    assert rel_l2(outs[0], ref["out"]) < 3e-3
    assert all(torch.equal(o, outs[0]) for o in outs[1:])       # partial sums are added in range order: no run-to-run noise
    plain = ops.linear_w8a8(xq, sx, dev(qw.view(torch.uint8)), dev(sw.view(-1)), dev(b), fmt, "e4m3", torch.bfloat16)
    assert rel_l2(outs[0], plain) < 3e-3


def test_splitk_argument_checks(ops):
    from dax_amd import _capi

    L = _capi.lib()
    assert L.daxq_linear_splitk_choice(75600, 5120, 5120) == 1 and L.daxq_linear_splitk_choice(256, 5120, 5120) == 2
    assert L.daxq_linear_splitk_choice(512, 5120, 5120) == 1     # 160 tiles: a second range would have to share CUs
    assert L.daxq_linear_splitk_choice(64, 5120, 5120) == 1
    need = L.daxq_linear_splitk_workspace_bytes(512, 5120, 2)
    assert need == 16384 + 160 * 2 * 65536      # the counter head (fixed) + two partial results for each of 160 tiles
    xq = torch.zeros(512, 1024, dtype=torch.int8, device="cuda")
    wq = torch.zeros(256, 1024, dtype=torch.int8, device="cuda")
    ones_m, ones_n = torch.ones(512, device="cuda"), torch.ones(256, device="cuda")
    out = torch.empty(512, 256, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(2 << 20, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (0, 0, xq.data_ptr(), 1024, ones_m.data_ptr(), wq.data_ptr(), 1024, ones_n.data_ptr(), None, out.data_ptr(), 256, 512, 256, 1024)
    assert L.daxq_linear_w8a8_splitk(*args, 2, ws.data_ptr(), 1000, st) == -1 and "workspace" in _capi.last_error()
    assert L.daxq_linear_w8a8_splitk(*args, 3, ws.data_ptr(), ws.numel(), st) == -2        # 8 units of K do not divide by 3
    assert L.daxq_linear_w8a8_splitk(*args, 2, ws.data_ptr() + 16, ws.numel() - 16, st) == -2
    assert L.daxq_linear_w8a8_splitk(*args, 2, ws.data_ptr(), ws.numel(), st) == 0
    torch.cuda.synchronize()
    assert bool((out == 0).all()) and bool((ws[:16384] == 0).all())
