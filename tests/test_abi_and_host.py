"""CPU-only checks: the C-ABI library loads and exports what include/daxq.h declares, and the host
side of the DAX module-swap API (qscheme, qconfig resolution, swap rules, constructor validation,
state layout, fake kernels) behaves like the reference describes.  No GPU compute is called."""
import ctypes
import os
import re

import pytest
import torch
from torch import nn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "daxq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(daxq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from dax_amd import _capi

    lib = ctypes.CDLL(_capi.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 12
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/daxq.h but not exported"
    assert set(declared) == set(_capi.SIGNATURES), "binding table and header disagree"
    assert _capi.lib().daxq_abi_version() == _capi.ABI_VERSION == 5
    assert "undefined symbol" not in _capi.last_error()


def test_header_is_plain_c_and_a_c_program_links(tmp_path):
    """include/daxq.h is the boundary a cgo / JNI / FFI binding would consume: it must compile as C99 and as C++11
    without extensions, and a C program that includes it must link against the library and run (only entry points that
    need no device are called)."""
    import shutil
    import subprocess

    from dax_amd import _capi

    gcc, gxx = shutil.which("gcc"), shutil.which("g++")
    if not gcc or not gxx:
        pytest.skip("no host compiler")
    src = tmp_path / "abi.c"
    src.write_text('#include <stdio.h>\n#include "daxq.h"\n'
                   "int main(void) {\n"
                   "    int (*f)(int, int, int, const void*, int64_t, const float*, const void*, int64_t, const float*, const void*,\n"
                   "             void*, int64_t, void*, int64_t, int64_t, int64_t, int64_t, int, daxq_stream_t) = daxq_linear_w8a8;\n"
                   '    printf("%d %d %s\\n", daxq_abi_version(), DAXQ_ABI_VERSION, f ? "ok" : "null");\n'
                   "    return daxq_abi_version() == DAXQ_ABI_VERSION ? 0 : 1;\n}\n")
    inc = os.path.join(ROOT, "include")
    subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", inc, str(src)], check=True)
    subprocess.run([gxx, "-std=c++11", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-x", "c++", "-I", inc, str(src)], check=True)
    exe = tmp_path / "abi"
    libdir = os.path.dirname(_capi.LIB_PATH)
    subprocess.run([gcc, "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-ldaxq", f"-Wl,-rpath,{libdir}",
                    "-Wl,--allow-shlib-undefined"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert out == [str(_capi.ABI_VERSION), str(_capi.ABI_VERSION), "ok"]


def test_patch_tile_order_covers_every_tile_once():
    """tests/host/tile_order_check (built by __graft_entry__.build() from the header the kernels include): every tile
    grid up to 320 x 72 and sampled grids up to 100003 tile rows and 4096 tile columns (the range the library's choice
    by shape admits), every tile exactly once, an XCD's 32 slots inside one patch."""
    import subprocess

    exe = os.path.join(ROOT, "tests", "host", "tile_order_check")
    if not os.path.exists(exe):     # a tree that was never built: one second of g++
        import __graft_entry__

        __graft_entry__._build_host_checks()
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and " 0 errors" in r.stdout, r.stdout + r.stderr


def test_tile_order_by_shape():
    """daxq_linear_tile_order_choice (host arithmetic only): the four Wan2.1-14B launches at 75600 tokens and their
    neighbours take the banded order; a 1/8 share of the rows, short K, narrow N and small launches keep the row
    groups."""
    from dax_amd import _capi

    f = _capi.lib().daxq_linear_tile_order_choice
    for n, k in ((15360, 5120), (5120, 5120), (13824, 5120), (5120, 13824)):
        assert f(75600, n, k) == 2
        assert all(f(m, n, k) == 2 for m in range(63488, 75777, 512))
        assert f(9450, n, k) == 1            # one XCD would end a whole patch ahead of its share
    assert f(32760, 15360, 5120) == 2 and f(20000, 15360, 5120) == 2
    assert f(75600, 5120, 1536) == 1         # K below 2048
    assert f(65536, 4096, 4096) == 1         # fewer than five bands
    assert f(4096, 15360, 5120) == 1         # less than one super-row of patches
    assert f(512, 5120, 5120) == 1 and f(1, 8, 128) == 1 and f(0, 0, 0) == 1


def test_kernel_argument_fields():
    """The host-side selection (tests, comparisons) packs the fields of the `kernel` argument as include/daxq.h lays
    them out: implementation in the low 16 bits, group depth in bits 16-23, tile order in 24-27, treatment of the last
    partial round of workgroups in 28-29."""
    from dax_amd import _capi

    try:
        for v in (8, 1005, 2002, 3002):
            _capi.debug_select_gemm(v)
        assert _capi.kernel_arg() == 8 | (5 << 16) | (2 << 24) | (2 << 28)
        for bad in (3, 6, 9, 1064, 2003, 3003, -1):
            with pytest.raises(_capi.DaxqError):
                _capi.debug_select_gemm(bad)
    finally:
        for v in (0, 1000, 2000, 3000):
            _capi.debug_select_gemm(v)
    assert _capi.kernel_arg() == 0


def test_no_cpu_kernels_and_clear_errors():
    import dax_amd.ops as ops

    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    for fn in (ops.act_quant_i8, ops.act_quant_e4m3, ops.row_minmax):
        with pytest.raises(NotImplementedError):
            fn(x)
    with pytest.raises(NotImplementedError):
        ops.linear_i8(torch.zeros(4, 128, dtype=torch.int8), torch.ones(4), torch.zeros(8, 128, dtype=torch.int8),
                      torch.ones(8), None)


def test_fake_kernels_give_shapes_for_tracing():
    import dax_amd.ops as ops  # noqa: F401

    x = torch.empty(10, 200, dtype=torch.bfloat16, device="meta")
    q, s = torch.ops.daxq.act_quant_i8(x)
    assert q.shape == (10, 256) and q.dtype == torch.int8 and s.shape == (10,) and s.dtype == torch.float32
    q8, _ = torch.ops.daxq.act_quant_e4m3(x)
    assert q8.dtype == torch.uint8
    w = torch.empty(24, 256, dtype=torch.int8, device="meta")
    out = torch.ops.daxq.linear_i8(q, s, w, torch.empty(24, device="meta"), None)
    assert out.shape == (10, 24) and out.dtype == torch.bfloat16
    out, acc = torch.ops.daxq.linear_i8_acc(q, s, w, torch.empty(24, device="meta"), None)
    assert acc.dtype == torch.int32 and acc.shape == (10, 24)
    qw = torch.ops.daxq.quantize_rows_i8(x, torch.empty(10, device="meta"), True)
    assert qw.shape == (10, 256)


def test_get_block_size_and_reduction_params():
    from dax_amd.quant.nn.dynamic.functional import _get_reduction_params
    from dax_amd.quant.qscheme import (get_block_size, per_channel_symmetric, per_tensor_symmetric,
                                       per_token_symmetric)

    assert per_token_symmetric == "dax.quant.per_token_symmetric"
    assert get_block_size((2, 3, 8), per_token_symmetric) == (1, 1, 8)
    assert get_block_size((2, 3, 8), per_tensor_symmetric) == (2, 3, 8)
    assert get_block_size((4, 8), per_channel_symmetric) == (4, 1)
    with pytest.raises(ValueError):
        get_block_size((4, 8), "nope")
    # the worked example of the reference docstring (dynamic/functional.py:20-27)
    assert _get_reduction_params((3, 3, 2, 10), (3, 3, 10, 10)) == ([3, 3, 5, 2, 10], [0, 1, 3, 4])
    assert _get_reduction_params((1, 8), (5, 8)) == ([5, 8], [1])
    with pytest.raises(AssertionError):
        _get_reduction_params((3,), (10,))


class Inner(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(8, 8)
        self.act = nn.ReLU()


class Outer(nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = Inner()
        self.block = Inner()
        self.proj_out = nn.Linear(8, 4)


class Sub(nn.Linear):
    pass


class FakeQ(nn.Module):
    """Stands in for the quantised module so the swap machinery can be exercised without a GPU."""
    made = []

    def __init__(self, src):
        super().__init__()
        self.src_shape = tuple(src.weight.shape)

    @classmethod
    def from_float(cls, mod, reserve_float_weight=False):
        FakeQ.made.append(mod)
        return cls(mod)


def _cfg():
    from dax_amd.quant.quantization.qconfig import get_dynamic_int8_per_token_act_per_channel_weight_qconfig

    return get_dynamic_int8_per_token_act_per_channel_weight_qconfig()


def test_qconfig_resolution_prefix_type_attr_and_inheritance():
    from dax_amd.quant.quantization.quantize import propagate_qconfig_

    m = Outer()
    cfg, other = _cfg(), _cfg()
    m.block.act.qconfig = other          # an existing attribute wins
    propagate_qconfig_(m, {"": cfg, "embed": None})
    assert m.qconfig is cfg and m.block.qconfig is cfg and m.block.fc.qconfig is cfg
    assert m.embed.qconfig is None and m.embed.fc.qconfig is None      # the subtree inherits None
    assert m.block.act.qconfig is other
    m2 = Outer()
    propagate_qconfig_(m2, {nn.Linear: cfg})                           # keyed by type
    assert m2.qconfig is None and m2.block.fc.qconfig is cfg and m2.proj_out.qconfig is cfg
    m3 = Outer()
    propagate_qconfig_(m3, {"": cfg, "block.fc": None})                # dotted child name
    assert m3.block.fc.qconfig is None and m3.embed.fc.qconfig is cfg
    with pytest.raises(AssertionError):
        propagate_qconfig_(Outer(), {"": object()})


def test_swap_rules_exact_type_none_subtree_hooks_and_cleanup():
    from dax_amd.quant.quantization import quantize_dynamic

    FakeQ.made.clear()
    m = Outer()
    m.block.sub = Sub(8, 8)              # a subclass of nn.Linear is not swapped
    seen = []
    m.block.fc.register_forward_pre_hook(lambda mod, inp: seen.append("pre"))
    m.block.fc.register_forward_hook(lambda mod, inp, out: seen.append("post"))
    out = quantize_dynamic(m, {"": _cfg(), "embed": None, "proj_out": None}, mapping={nn.Linear: FakeQ})
    assert out is m                                                    # in place by default
    assert isinstance(m.block.fc, FakeQ) and m.block.fc.src_shape == (8, 8)
    assert type(m.embed.fc) is nn.Linear and type(m.proj_out) is nn.Linear and type(m.block.sub) is Sub
    assert len(FakeQ.made) == 1
    assert len(m.block.fc._forward_pre_hooks) == 1 and len(m.block.fc._forward_hooks) == 1
    assert not any(hasattr(mod, "qconfig") for mod in m.modules())     # remove_qconfig=True
    m2 = Outer()
    q2 = quantize_dynamic(m2, {"": _cfg()}, mapping={nn.Linear: FakeQ}, inplace=False, remove_qconfig=False)
    assert q2 is not m2 and type(m2.block.fc) is nn.Linear and isinstance(q2.block.fc, FakeQ)
    assert hasattr(q2.block, "qconfig")


def test_default_mappings_and_prepare_convert_flow():
    from dax_amd.quant.nn import dynamic, quantized
    from dax_amd.quant.quantization import convert, prepare
    from dax_amd.quant.quantization.qconfig import get_default_fp8_qconfig
    from dax_amd.quant.quantization.quantization_mappings import (get_default_dynamic_quant_module_mappings,
                                                                  get_default_qconfig_propagation_list,
                                                                  get_default_static_quant_module_mappings)
    from dax_amd.quant.quantization.observer import MinMaxObserver
    from dax_amd.quant.quantization.quantize import _observer_forward_pre_hook

    assert get_default_dynamic_quant_module_mappings() == {nn.Linear: dynamic.Linear}
    assert get_default_static_quant_module_mappings() == {nn.Linear: quantized.Linear}
    assert get_default_qconfig_propagation_list() == {nn.Linear}
    # prepare: observers on the leaf linears that have a qconfig, as the first pre-hook; nowhere else
    m = Outer()
    user_hook = lambda mod, inp: None
    m.block.fc.register_forward_pre_hook(user_hook)
    prepare(m, {"": get_default_fp8_qconfig(), "embed": None})
    assert isinstance(m.block.fc.activation_post_process, MinMaxObserver)
    assert list(m.block.fc._forward_pre_hooks.values())[0] is _observer_forward_pre_hook
    assert not hasattr(m.embed.fc, "activation_post_process") and not hasattr(m.block, "activation_post_process")
    assert m.block.fc.activation_post_process.calculate_qparams() is None      # nothing observed yet
    # convert with a stand-in target: the observer hook does not travel, the user's hook does, clean-up is complete
    FakeQ.made.clear()
    convert(m, mapping={nn.Linear: FakeQ})
    assert isinstance(m.block.fc, FakeQ) and type(m.embed.fc) is nn.Linear
    assert list(m.block.fc._forward_pre_hooks.values()) == [user_hook]
    assert not any(hasattr(mod, "qconfig") or hasattr(mod, "activation_post_process") for mod in m.modules())
    # observer_non_leaf_module_list: a listed non-leaf child is observed as a whole and not descended into
    # (dax/quant/quantization/quantize.py:205-210)
    m = Outer()
    prepare(m, {"": get_default_fp8_qconfig(), "embed": None}, observer_non_leaf_module_list=[Inner])
    assert isinstance(m.block.activation_post_process, MinMaxObserver)
    assert list(m.block._forward_pre_hooks.values())[0] is _observer_forward_pre_hook
    assert not hasattr(m.block.fc, "activation_post_process")           # not descended into
    assert not hasattr(m.embed, "activation_post_process")              # its qconfig is None
    assert isinstance(m.proj_out.activation_post_process, MinMaxObserver)  # leaves elsewhere as before


def test_static_linear_state_and_validation():
    from dax_amd.quant.nn.quantized import Linear

    lin = Linear(64, 32, True, None, torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16, row_wise_scale=False)
    sd = lin.state_dict()
    assert set(sd) == {"qweight", "weight_scale", "input_scale", "bias"}
    assert sd["weight_scale"].shape == (1,) and sd["input_scale"].shape == (1,) and sd["qweight"].dtype == torch.float8_e4m3fn
    assert Linear(64, 32, False, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.bfloat16, True).weight_scale.shape == (1, 32)
    assert "input_scale" in lin.extra_repr()
    e5 = Linear(8, 8, True, None, torch.float8_e5m2, torch.float8_e5m2, torch.float16)     # e5m2 weights, fp16 module
    assert e5.qweight.dtype == torch.float8_e5m2 and e5.bias.dtype == torch.float16 and e5.out_dtype == torch.float16
    assert Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.float32, True).bias.dtype == torch.bfloat16
    with pytest.raises(NotImplementedError):
        Linear(8, 8, True, None, torch.float8_e4m3fn, torch.int8, torch.bfloat16)
    with pytest.raises(ValueError, match="Input must be quantized"):
        Linear.get_qlinear(nn.Linear(8, 8), None, None, False)
    with pytest.raises(AssertionError):
        Linear.from_float(Sub(8, 8))


def test_linear_constructor_validation_and_state_layout():
    from dax_amd.quant.nn.dynamic import Linear
    from dax_amd.quant.qscheme import per_channel_symmetric as ch, per_tensor_symmetric as te, per_token_symmetric as tok

    lin = Linear(256, 128, True, None, torch.int8, torch.int8, torch.bfloat16, ch, tok)
    sd = lin.state_dict()
    assert set(sd) == {"qweight", "weight_scale", "bias"}
    assert sd["qweight"].shape == (128, 256) and sd["qweight"].dtype == torch.int8
    assert sd["weight_scale"].shape == (1, 128) and sd["weight_scale"].dtype == torch.float32
    assert sd["bias"].dtype == torch.bfloat16 and lin.compute_dtype == "INT8"
    assert "in_features=256, out_features=128" in lin.extra_repr() and lin._FLOAT_MODULE is nn.Linear
    f8 = Linear(64, 32, False, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.bfloat16, ch, tok)
    assert f8.compute_dtype == "FP8" and f8.bias is None and f8.qweight.dtype == torch.float8_e4m3fn
    assert "bias=False" in f8.extra_repr()
    with pytest.raises(ValueError):      # mixed int8 / fp8
        Linear(8, 8, True, None, torch.int8, torch.float8_e4m3fn, torch.bfloat16, ch, tok)
    with pytest.raises(ValueError):      # fp8 with a qscheme pair the reference rejects
        Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.bfloat16, ch, te)
    with pytest.raises(ValueError):
        Linear(8, 8, True, None, torch.float32, torch.float32, torch.bfloat16, ch, tok)
    pt = Linear(8, 16, True, None, torch.int8, torch.int8, torch.bfloat16, te, te)       # per-tensor pair
    assert pt.weight_scale.shape == (1,) and pt.input_qscheme == te
    assert Linear(8, 16, True, None, torch.int8, torch.int8, torch.bfloat16, ch, te).weight_scale.shape == (1, 16)
    assert Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16, te, te).compute_dtype == "FP8"
    mixed = Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16, ch, tok)
    assert mixed.compute_dtype == "FP8" and mixed.input_dtype == torch.float8_e5m2   # the reference's FP8 default
    e5 = Linear(8, 8, True, None, torch.float8_e5m2, torch.float8_e5m2, torch.bfloat16, ch, tok)   # e5m2 weights
    assert e5.qweight.dtype == torch.float8_e5m2 and e5.compute_dtype == "FP8"
    # module dtypes other than bf16 (out_dtype = the float weight's dtype, dax/quant/nn/dynamic/linear.py:263): the bias is
    # kept in that dtype, except for the row-wise FP8 matmul, which takes a bf16 bias (:106-118)
    assert Linear(8, 8, True, None, torch.int8, torch.int8, torch.float16, ch, tok).bias.dtype == torch.float16
    assert Linear(8, 8, True, None, torch.int8, torch.int8, torch.float32, ch, tok).bias.dtype == torch.float32
    assert Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.float16, ch, tok).bias.dtype == torch.bfloat16
    assert Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e4m3fn, torch.float16, te, te).bias.dtype == torch.float16
    with pytest.raises(NotImplementedError):
        Linear(8, 8, True, None, torch.int8, torch.int8, torch.float64, ch, tok)
    # dequantised weight property is plain tensor algebra on the stored state
    with torch.no_grad():
        lin.qweight.copy_(torch.randint(-127, 128, (128, 256), dtype=torch.int8))
        lin.weight_scale.copy_(torch.rand(1, 128) * 0.01)
    w = lin.weight
    assert w.shape == (128, 256) and w.dtype == torch.bfloat16
    assert torch.equal(w, lin.qweight.bfloat16() * lin.weight_scale.T.bfloat16())


def test_from_float_asserts_and_loud_failure_without_gpu():
    from dax_amd.quant.nn.dynamic import Linear

    with pytest.raises(AssertionError):
        Linear.from_float(Sub(8, 8))
    with pytest.raises(AssertionError):
        Linear.from_float(nn.Linear(8, 8))             # no qconfig
    lin = nn.Linear(8, 8).bfloat16()
    lin.qconfig = _cfg()
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no ROCm device"):
            Linear.from_float(lin)
    from dax_amd.quant.quantization.observer import DynamicObserverPlaceholder

    with pytest.raises(ValueError, match="Input must be quantized"):
        Linear.get_qlinear(nn.Linear(8, 8), None, _cfg().weight(), False)
    ph = DynamicObserverPlaceholder(dtype=torch.int8, qscheme="dax.quant.per_token_symmetric", is_dynamic=True)
    assert ph.quant_max == 127 and ph.forward(torch.zeros(1)) is None and float(ph.eps) == 2.0 ** -23


def test_qconfig_factories_defaults():
    from dax_amd.quant.qscheme import per_channel_symmetric, per_token_symmetric
    from dax_amd.quant.quantization.qconfig import (get_dynamic_fp8_per_token_act_per_channel_weight_qconfig as f8,
                                                    get_dynamic_int8_per_token_act_per_channel_weight_qconfig as i8)

    c = i8()
    a, w = c.activation(), c.weight()
    assert a.dtype == torch.int8 and a.qscheme == per_token_symmetric and a.is_dynamic
    assert w.dtype == torch.int8 and w.qscheme == per_channel_symmetric and w.quant_max == 127
    c8 = f8()
    assert c8.activation().dtype == torch.float8_e5m2         # the reference's default
    assert c8.weight().dtype == torch.float8_e4m3fn and c8.weight().quant_max == 448.0
    assert f8(activation_dtype=torch.float8_e4m3fn).activation().dtype == torch.float8_e4m3fn
    assert w.calculate_qparams() is None                       # nothing observed yet
    from dax_amd.quant.qscheme import per_tensor_symmetric
    from dax_amd.quant.quantization import qconfig as Q
    from dax_amd.quant.quantization.observer import MinMaxObserver, PerChannelMinMaxObserver

    for fac, act_dyn, act_scheme, w_cls, a_dt in [
        (Q.get_default_fp8_qconfig, False, per_tensor_symmetric, MinMaxObserver, torch.float8_e5m2),
        (Q.get_fp8_per_channel_weight_qconfig, False, per_tensor_symmetric, PerChannelMinMaxObserver, torch.float8_e5m2),
        (Q.get_default_dynamic_fp8_qconfig, True, per_tensor_symmetric, MinMaxObserver, torch.float8_e5m2),
        (Q.get_default_dynamic_int8_qconfig, True, per_tensor_symmetric, MinMaxObserver, torch.int8),
        (Q.get_dynamic_int8_per_channel_weight_qconfig, True, per_tensor_symmetric, PerChannelMinMaxObserver, torch.int8),
    ]:
        cfg = fac()
        act, wt = cfg.activation(), cfg.weight()
        assert act.is_dynamic == act_dyn and act.qscheme == act_scheme and act.dtype == a_dt and isinstance(wt, w_cls)
        if not act_dyn:
            assert isinstance(act, MinMaxObserver) and act.sync_state
    with pytest.raises(NotImplementedError):
        Q.get_default_dist_profile_qconfig()


def test_optimize_pipe_switches():
    from dax_amd.adapters.wan import optimize_pipe

    class Pipe:
        transformer = nn.Sequential()

    with pytest.raises(NotImplementedError):
        optimize_pipe(Pipe(), sequence_parallel=True)
    with pytest.raises(ValueError):
        optimize_pipe(Pipe(), int8_linear=True, fp8_linear=True)
    p = Pipe()
    assert optimize_pipe(p) is p


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys

    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_block_fusion_host_logic_without_gpu():
    """fuse_linears layout, what counts as a fusable block, and that the new ops are declared."""
    import torch
    from dax_amd.adapters.wan import block_fusion as BF
    from dax_amd.quant.nn.dynamic import Linear, QuantizedActivation
    from dax_amd.quant.qscheme import per_channel_symmetric, per_token_symmetric
    from tests.wan_replica import Transformer

    def lin(n, k, seed):
        l = Linear(k, n, True, None, torch.int8, torch.int8, torch.bfloat16, per_channel_symmetric, per_token_symmetric)
        g = torch.Generator().manual_seed(seed)
        l.qweight.copy_(torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8))
        l.weight_scale.copy_(torch.rand(1, n, generator=g) + 0.1)
        with torch.no_grad():
            l.bias.copy_(torch.randn(n, generator=g))
        return l

    a, b = lin(8, 16, 0), lin(24, 16, 1)
    f = BF.fuse_linears([a, b])
    assert f.out_features == 32 and torch.equal(f.qweight[:8], a.qweight) and torch.equal(f.qweight[8:], b.qweight)
    assert torch.equal(f.weight_scale[:, 8:], b.weight_scale) and torch.equal(f.bias[:8], a.bias)
    assert set(f.state_dict().keys()) == {"qweight", "weight_scale", "bias"}
    with pytest.raises(ValueError):
        BF.fuse_linears([a, lin(8, 32, 2)])                       # different in_features
    model = Transformer(dim=64, ffn_dim=128, heads=2, layers=1)
    assert not BF._block_is_fusable(model.blocks[0])              # float linears: nothing to fuse
    assert BF.fuse_transformer_blocks(model) == 0
    qa = QuantizedActivation(torch.zeros(6, 128, dtype=torch.int8), torch.ones(6), (2, 3), 16, torch.int8)
    assert qa.shape == (2, 3, 16)
    with pytest.raises(ValueError):
        lin(8, 32, 3)(qa)                                         # K mismatch is reported, not mis-computed


def test_prequantised_checkpoint_round_trip_from_a_meta_skeleton(tmp_path):
    """save_quantized / load_quantized: the file holds the reference's module state; loading builds the
    quantised modules from the qconfig on a meta skeleton and copies, no kernel involved (runs on the CPU)."""
    from dax_amd.quant.checkpoint import load_quantized, save_quantized
    from dax_amd.quant.nn import dynamic, quantized
    from dax_amd.quant.qscheme import per_channel_symmetric, per_token_symmetric
    from dax_amd.quant.quantization.qconfig import get_default_fp8_qconfig

    src = Outer()
    g = torch.Generator().manual_seed(0)
    q = dynamic.Linear(8, 8, True, None, torch.int8, torch.int8, torch.bfloat16, per_channel_symmetric, per_token_symmetric)
    q.qweight.copy_(torch.randint(-127, 128, (8, 8), generator=g, dtype=torch.int8))
    q.weight_scale.copy_(torch.rand(1, 8, generator=g))
    with torch.no_grad():
        q.bias.copy_(torch.randn(8, generator=g))
    src.block.fc = q
    path = str(tmp_path / "m.safetensors")
    save_quantized(src, path)
    with torch.device("meta"):
        skel = Outer()
    out = load_quantized(skel, path, {"block": _cfg()}, device="cpu")
    assert isinstance(out.block.fc, dynamic.Linear) and type(out.embed.fc) is nn.Linear
    assert not any(p.device.type == "meta" for p in out.parameters())
    for k, v in src.state_dict().items():
        assert torch.equal(out.state_dict()[k].view(torch.uint8) if v.dtype == torch.int8 else out.state_dict()[k], 
                           v.view(torch.uint8) if v.dtype == torch.int8 else v), k
    assert not any(hasattr(m, "qconfig") for m in out.modules())
    # a static qconfig gives the static module (fp8 tensors are stored natively in the file)
    s = Outer()
    st = quantized.Linear(8, 8, True, None, torch.float8_e4m3fn, torch.float8_e5m2, torch.bfloat16, False)
    with torch.no_grad():
        st.qweight.copy_(torch.randn(8, 8, generator=g).to(torch.float8_e4m3fn))
        st.input_scale.fill_(0.25)
        st.bias.zero_()
    s.block.fc = st
    save_quantized(s, path)
    with torch.device("meta"):
        skel2 = Outer()
    out2 = load_quantized(skel2, path, {"block": get_default_fp8_qconfig()}, device="cpu")
    assert isinstance(out2.block.fc, quantized.Linear) and float(out2.block.fc.input_scale) == 0.25
    assert torch.equal(out2.block.fc.qweight.view(torch.uint8), st.qweight.view(torch.uint8))
    with pytest.raises(RuntimeError):                         # a skeleton that does not match the file is reported
        with torch.device("meta"):
            bad = Outer()
        load_quantized(bad, path, {}, device="cpu")


@pytest.mark.parametrize("k", [384, 392])
@pytest.mark.parametrize("dtype", [torch.int8, torch.float8_e4m3fn])
def test_module_forward_traces_with_fake_tensors(dtype, k):
    """Shape and dtype propagation through the fake kernels, as a tracer sees the module: no device, no
    kernel call.  Also the per-tensor forms, whose scale vectors come from further ops."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    from dax_amd.quant.nn.dynamic.linear import Linear
    from dax_amd.quant.qscheme import per_channel_symmetric, per_tensor_symmetric, per_token_symmetric

    for in_s, w_s in [(per_token_symmetric, per_channel_symmetric), (per_tensor_symmetric, per_tensor_symmetric)]:
        with FakeTensorMode():
            lin = Linear(k, 520, device="cuda", weight_dtype=dtype, input_dtype=dtype, weight_qscheme=w_s,
                         input_qscheme=in_s)
            qa = lin.quantize_activation(torch.empty(2, 300, k, dtype=torch.bfloat16, device="cuda"))
            assert qa.xq.shape == (600, (k + 127) // 128 * 128) and qa.sx.shape == (600,) and qa.sx.dtype == torch.float32
            y = lin(torch.empty(2, 300, k, dtype=torch.bfloat16, device="cuda"))
            assert y.shape == (2, 300, 520) and y.dtype == torch.bfloat16 and y.device.type == "cuda"


def test_product_never_touches_the_oracle_or_a_cpu_path():
    """The oracle is test infrastructure: no file of the package names it, and every custom op is registered for
    the GPU only."""
    pkg = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "dax_amd")
    for root, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".c", ".cpp")):
                text = open(os.path.join(root, f), errors="ignore").read()
                assert not re.search(r"\boracle\b", text), f"{os.path.join(root, f)} mentions the oracle"
    ops_src = open(os.path.join(pkg, "ops.py")).read()
    decls = [line for line in ops_src.splitlines() if line.startswith("@torch.library.custom_op(")]
    assert decls and all('device_types="cuda"' in d for d in decls)


def test_bench_inputs_follow_the_seeded_recipe():
    """bench.py generates its operands with the oracle's seeded CPU recipe (the column scaling is written as one
    multiplication by a vector there): same bits."""
    import bench
    from oracle import daxq_oracle as O

    for seed, (m, k, n) in enumerate([(64, 1536, 24), (33, 200, 8)]):
        a, b = bench.synth_inputs(m, k, n, seed), O.make_inputs(m, k, n, seed)
        assert all(torch.equal(u, v) and u.dtype == torch.bfloat16 for u, v in zip(a, b))
