"""``torch.ops.daxq.*``: the HIP kernels of libdaxq as PyTorch custom ops.

Each op allocates its outputs with torch (device memory is torch's), passes raw device
pointers and the current HIP stream through the C ABI, and has a fake (meta) kernel so a
surrounding ``torch.compile`` graph can trace through it.  No op has a CPU kernel.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _capi

K_ALIGN = 128  # DAXQ_K_ALIGN


def pad_k(k: int) -> int:
    return (k + K_ALIGN - 1) // K_ALIGN * K_ALIGN


def is_tracing(t: torch.Tensor) -> bool:
    """True while a graph is being traced over ``t``: it has no storage address to key a cache on."""
    from torch._subclasses.fake_tensor import FakeTensor

    return torch.compiler.is_compiling() or isinstance(t, FakeTensor)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """The HIP stream that is current for the tensor's device, as an integer handle."""
    idx = t.device.index
    if _raw_stream is not None and idx is not None:
        return _raw_stream(idx)  # the same handle without building a Stream object (a tenth of the host time)
    return torch.cuda.current_stream(t.device).cuda_stream


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _on_device(t: torch.Tensor):
    """Context that makes the tensor's device current for the allocations and the launch; with a single GPU it is
    current already and the guard (several microseconds per call) is left out."""
    return torch.cuda.device(t.device) if torch.cuda.device_count() > 1 else _NO_GUARD


def _need_gpu(t: torch.Tensor, what: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(f"daxq::{what}: tensor is on {t.device}; the daxq kernels only run on an MI355X "
                           "(there is no CPU implementation)")
    _capi.require_gfx950(t.device.index if t.device.index is not None else torch.cuda.current_device())


def _same_device(what: str, ref: torch.Tensor, **others) -> None:
    """Raises unless every given tensor lives on ref's device.  A custom op registered for "cuda" is dispatched as
    soon as one argument is a device tensor, so a module left on the CPU would otherwise hand host addresses to
    the kernels' loads."""
    for name, t in others.items():
        if t is not None and t.device != ref.device:
            raise ValueError(f"daxq::{what}: expected all tensors to be on the same device, but {name} is on {t.device} "
                             f"and the first operand on {ref.device}")


def _rows_bf16(x: torch.Tensor, what: str) -> None:
    _need_gpu(x, what)
    if x.dtype != torch.bfloat16:
        raise NotImplementedError(f"daxq::{what}: only bfloat16 inputs are implemented, got {x.dtype}")
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError(f"daxq::{what}: expected a 2-d tensor with contiguous rows, got shape {tuple(x.shape)} "
                         f"strides {x.stride()}")


# ----------------------------------------------------------------------------- act quant
def _act_quant(x: torch.Tensor, fp8, e5m2: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    name = "act_quant_e5m2" if e5m2 else "act_quant_e4m3" if fp8 else "act_quant_i8"
    _rows_bf16(x, name)
    m, k = x.shape
    kp = pad_k(k)
    with _on_device(x):
        q = torch.empty((m, kp), dtype=torch.uint8 if fp8 else torch.int8, device=x.device)
        s = torch.empty((m,), dtype=torch.float32, device=x.device)
        if m:
            fn = getattr(_capi.lib(), "daxq_" + name)
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(fn(x.data_ptr(), m, k, ld_x, q.data_ptr(), kp, s.data_ptr(), _stream(x)), name)
    return q, s


@torch.library.custom_op("daxq::act_quant_i8", mutates_args=(), device_types="cuda")
def act_quant_i8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [M,K] -> (int8 [M, pad128(K)] zero padded, fp32 [M] per-token scale)."""
    return _act_quant(x, False)


@torch.library.custom_op("daxq::act_quant_e4m3", mutates_args=(), device_types="cuda")
def act_quant_e4m3(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [M,K] -> (e4m3fn bytes as uint8 [M, pad128(K)], fp32 [M] per-token scale)."""
    return _act_quant(x, True)


@torch.library.custom_op("daxq::act_quant_e5m2", mutates_args=(), device_types="cuda")
def act_quant_e5m2(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [M,K] -> (e5m2 bytes as uint8 [M, pad128(K)], fp32 [M] per-token scale)."""
    return _act_quant(x, True, True)


def _act_quant_fake(x, dtype):
    return x.new_empty((x.shape[0], pad_k(x.shape[1])), dtype=dtype), x.new_empty((x.shape[0],), dtype=torch.float32)


act_quant_i8.register_fake(lambda x: _act_quant_fake(x, torch.int8))
act_quant_e4m3.register_fake(lambda x: _act_quant_fake(x, torch.uint8))
act_quant_e5m2.register_fake(lambda x: _act_quant_fake(x, torch.uint8))


# ----------------------------------------------------------------------------- producer + act quant
_FMT_NAMES = ("i8", "e4m3", "e5m2")


def _fused_out(x: torch.Tensor, fmt: str, want_y: bool):
    m, k = x.shape
    q = torch.empty((m, pad_k(k)), dtype=torch.int8 if fmt == "i8" else torch.uint8, device=x.device)
    s = torch.empty((m,), dtype=torch.float32, device=x.device)
    y = torch.empty((m, k) if want_y else (0, k), dtype=torch.bfloat16, device=x.device)
    return q, s, y


def _vec_arg(v: Optional[torch.Tensor], x: torch.Tensor, groups: int, what: str) -> int:
    if v is None:
        return 0
    if v.dtype != torch.float32 or v.device != x.device or not v.is_contiguous() or v.numel() != groups * x.shape[1]:
        raise ValueError(f"daxq::{what}: mul / add must be contiguous fp32 [{groups}, {x.shape[1]}] on {x.device}")
    return v.data_ptr()


def _layernorm_act_quant(fmt: str, x, mul, add, rows_per_group: int, eps: float, want_y: bool):
    name = "layernorm_act_quant_" + fmt
    _rows_bf16(x, name)
    m, k = x.shape
    if rows_per_group <= 0:
        raise ValueError(f"daxq::{name}: rows_per_group must be positive")
    groups = max(1, -(-m // rows_per_group))
    with _on_device(x):
        q, s, y = _fused_out(x, fmt, want_y)
        if m:
            fn = getattr(_capi.lib(), "daxq_" + name)
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(fn(x.data_ptr(), m, k, ld_x, _vec_arg(mul, x, groups, name), _vec_arg(add, x, groups, name),
                           rows_per_group, eps, y.data_ptr() if want_y else 0, k, q.data_ptr(), q.shape[1],
                           s.data_ptr(), _stream(x)), name)
    return q, s, y


def _gelu_tanh_act_quant(fmt: str, x, want_y: bool):
    name = "gelu_tanh_act_quant_" + fmt
    _rows_bf16(x, name)
    m, k = x.shape
    with _on_device(x):
        q, s, y = _fused_out(x, fmt, want_y)
        if m:
            fn = getattr(_capi.lib(), "daxq_" + name)
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(fn(x.data_ptr(), m, k, ld_x, y.data_ptr() if want_y else 0, k, q.data_ptr(), q.shape[1],
                           s.data_ptr(), _stream(x)), name)
    return q, s, y


def _fused_fake(x, fmt, want_y):
    return (x.new_empty((x.shape[0], pad_k(x.shape[1])), dtype=torch.int8 if fmt == "i8" else torch.uint8),
            x.new_empty((x.shape[0],), dtype=torch.float32),
            x.new_empty((x.shape[0] if want_y else 0, x.shape[1]), dtype=torch.bfloat16))


@torch.library.custom_op("daxq::layernorm_act_quant_i8", mutates_args=(), device_types="cuda")
def layernorm_act_quant_i8(x: torch.Tensor, mul: Optional[torch.Tensor], add: Optional[torch.Tensor],
                           rows_per_group: int, eps: float,
                           want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = bf16(layer_norm_f32(x, eps) * mul[row // rows_per_group] + add[...]) and its per-token int8
    quantisation in one pass: (q [M, pad128(K)], scale [M], y [M, K] or an empty [0, K])."""
    return _layernorm_act_quant("i8", x, mul, add, rows_per_group, eps, want_y)


@torch.library.custom_op("daxq::layernorm_act_quant_e4m3", mutates_args=(), device_types="cuda")
def layernorm_act_quant_e4m3(x: torch.Tensor, mul: Optional[torch.Tensor], add: Optional[torch.Tensor],
                             rows_per_group: int, eps: float,
                             want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _layernorm_act_quant("e4m3", x, mul, add, rows_per_group, eps, want_y)


@torch.library.custom_op("daxq::layernorm_act_quant_e5m2", mutates_args=(), device_types="cuda")
def layernorm_act_quant_e5m2(x: torch.Tensor, mul: Optional[torch.Tensor], add: Optional[torch.Tensor],
                             rows_per_group: int, eps: float,
                             want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _layernorm_act_quant("e5m2", x, mul, add, rows_per_group, eps, want_y)


@torch.library.custom_op("daxq::gelu_tanh_act_quant_i8", mutates_args=(), device_types="cuda")
def gelu_tanh_act_quant_i8(x: torch.Tensor, want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """y = bf16(gelu(x, approximate="tanh")) and its per-token int8 quantisation in one pass."""
    return _gelu_tanh_act_quant("i8", x, want_y)


@torch.library.custom_op("daxq::gelu_tanh_act_quant_e4m3", mutates_args=(), device_types="cuda")
def gelu_tanh_act_quant_e4m3(x: torch.Tensor, want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _gelu_tanh_act_quant("e4m3", x, want_y)


@torch.library.custom_op("daxq::gelu_tanh_act_quant_e5m2", mutates_args=(), device_types="cuda")
def gelu_tanh_act_quant_e5m2(x: torch.Tensor, want_y: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    return _gelu_tanh_act_quant("e5m2", x, want_y)


layernorm_act_quant_i8.register_fake(lambda x, mul, add, rows_per_group, eps, want_y=False: _fused_fake(x, "i8", want_y))
layernorm_act_quant_e4m3.register_fake(lambda x, mul, add, rows_per_group, eps, want_y=False: _fused_fake(x, "e4m3", want_y))
layernorm_act_quant_e5m2.register_fake(lambda x, mul, add, rows_per_group, eps, want_y=False: _fused_fake(x, "e5m2", want_y))
gelu_tanh_act_quant_i8.register_fake(lambda x, want_y=False: _fused_fake(x, "i8", want_y))
gelu_tanh_act_quant_e4m3.register_fake(lambda x, want_y=False: _fused_fake(x, "e4m3", want_y))
gelu_tanh_act_quant_e5m2.register_fake(lambda x, want_y=False: _fused_fake(x, "e5m2", want_y))


# ----------------------------------------------------------------------------- leaf quantisers
def _quantize_rows(x: torch.Tensor, scale: torch.Tensor, fmt: str, padded: bool) -> torch.Tensor:
    name = "quantize_rows_" + fmt
    _rows_bf16(x, name)
    m, k = x.shape
    if scale.dtype != torch.float32 or scale.numel() != m or scale.device != x.device:
        raise ValueError(f"daxq::{name}: scale must be fp32 with one value per row on {x.device}")
    scale = scale.reshape(-1).contiguous()
    ld_q = pad_k(k) if padded else k
    with _on_device(x):
        q = torch.empty((m, ld_q), dtype=torch.int8 if fmt == "i8" else torch.uint8, device=x.device)
        if m:
            fn = getattr(_capi.lib(), "daxq_" + name)
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(fn(x.data_ptr(), m, k, ld_x, scale.data_ptr(), q.data_ptr(), ld_q, _stream(x)), name)
    return q


@torch.library.custom_op("daxq::quantize_rows_i8", mutates_args=(), device_types="cuda")
def quantize_rows_i8(x: torch.Tensor, scale: torch.Tensor, padded: bool = False) -> torch.Tensor:
    return _quantize_rows(x, scale, "i8", padded)


@torch.library.custom_op("daxq::quantize_rows_e4m3", mutates_args=(), device_types="cuda")
def quantize_rows_e4m3(x: torch.Tensor, scale: torch.Tensor, padded: bool = False) -> torch.Tensor:
    return _quantize_rows(x, scale, "e4m3", padded)


@torch.library.custom_op("daxq::quantize_rows_e5m2", mutates_args=(), device_types="cuda")
def quantize_rows_e5m2(x: torch.Tensor, scale: torch.Tensor, padded: bool = False) -> torch.Tensor:
    return _quantize_rows(x, scale, "e5m2", padded)


quantize_rows_e5m2.register_fake(
    lambda x, scale, padded=False: x.new_empty((x.shape[0], pad_k(x.shape[1]) if padded else x.shape[1]), dtype=torch.uint8))
quantize_rows_i8.register_fake(
    lambda x, scale, padded=False: x.new_empty((x.shape[0], pad_k(x.shape[1]) if padded else x.shape[1]), dtype=torch.int8))
quantize_rows_e4m3.register_fake(
    lambda x, scale, padded=False: x.new_empty((x.shape[0], pad_k(x.shape[1]) if padded else x.shape[1]), dtype=torch.uint8))


# ----------------------------------------------------------------------------- weight observer statistics
@torch.library.custom_op("daxq::row_minmax", mutates_args=(), device_types="cuda")
def row_minmax(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-row (min, max) of a bf16 matrix in fp32."""
    _rows_bf16(x, "row_minmax")
    m, k = x.shape
    with _on_device(x):
        lo = torch.empty((m,), dtype=torch.float32, device=x.device)
        hi = torch.empty((m,), dtype=torch.float32, device=x.device)
        if m:
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(_capi.lib().daxq_row_minmax(x.data_ptr(), m, k, ld_x, lo.data_ptr(), hi.data_ptr(), _stream(x)),
                        "row_minmax")
    return lo, hi


row_minmax.register_fake(lambda x: (x.new_empty((x.shape[0],), dtype=torch.float32),
                                    x.new_empty((x.shape[0],), dtype=torch.float32)))


@torch.library.custom_op("daxq::scale_from_minmax", mutates_args=(), device_types="cuda")
def scale_from_minmax(min_val: torch.Tensor, max_val: torch.Tensor, qmax: float) -> torch.Tensor:
    """max(max(-min, max) / qmax, 2^-23) element-wise in fp32."""
    _need_gpu(min_val, "scale_from_minmax")
    _same_device("scale_from_minmax", min_val, max_val=max_val)
    if min_val.dtype != torch.float32 or max_val.dtype != torch.float32 or min_val.shape != max_val.shape:
        raise ValueError("daxq::scale_from_minmax: min/max must be fp32 tensors of one shape")
    lo, hi = min_val.contiguous(), max_val.contiguous()
    with _on_device(lo):
        s = torch.empty_like(lo)
        _capi.check(_capi.lib().daxq_scale_from_minmax(lo.data_ptr(), hi.data_ptr(), lo.numel(), float(qmax),
                                                       s.data_ptr(), _stream(lo)), "scale_from_minmax")
    return s


scale_from_minmax.register_fake(lambda min_val, max_val, qmax: torch.empty_like(min_val))


# ----------------------------------------------------------------------------- GEMM + epilogue
def _linear(xq, sx, wq, sw, bias, fp8: bool, want_acc: bool, x_e5m2: bool = False):
    name = "linear_e5m2_e4m3" if x_e5m2 else "linear_e4m3" if fp8 else "linear_i8"
    _need_gpu(xq, name)
    _same_device(name, xq, sx=sx, wq=wq, sw=sw, bias=bias)
    qdt = torch.uint8 if fp8 else torch.int8
    if xq.dtype != qdt or wq.dtype != qdt:
        raise ValueError(f"daxq::{name}: operands must be {qdt}")
    if xq.dim() != 2 or wq.dim() != 2 or xq.stride(1) != 1 or wq.stride(1) != 1 or xq.shape[1] != wq.shape[1]:
        raise ValueError(f"daxq::{name}: expected xq [M,Kp] and wq [N,Kp] with contiguous rows, got "
                         f"{tuple(xq.shape)} and {tuple(wq.shape)}")
    m, k = xq.shape
    n = wq.shape[0]
    if sx.dtype != torch.float32 or sw.dtype != torch.float32 or sx.numel() != m or sw.numel() != n:
        raise ValueError(f"daxq::{name}: sx must be fp32 [M] and sw fp32 [N]")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n):
        raise ValueError(f"daxq::{name}: bias must be bf16 [N]")
    sx = sx.reshape(-1).contiguous()
    sw = sw.reshape(-1).contiguous()
    bias_c = bias.contiguous() if bias is not None else None
    with _on_device(xq):
        out = torch.empty((m, n), dtype=torch.bfloat16, device=xq.device)
        acc = torch.empty((m, n), dtype=torch.float32 if fp8 else torch.int32, device=xq.device) if want_acc else None
        if m and n:
            fn = getattr(_capi.lib(), "daxq_" + name)
            ld_x = xq.stride(0) if m > 1 else k
            ld_w = wq.stride(0) if n > 1 else k
            _capi.check(fn(xq.data_ptr(), ld_x, sx.data_ptr(), wq.data_ptr(), ld_w, sw.data_ptr(),
                           bias_c.data_ptr() if bias_c is not None else None, out.data_ptr(), n,
                           acc.data_ptr() if acc is not None else None, n, m, n, k, _stream(xq)), name)
    return out, acc


@torch.library.custom_op("daxq::linear_i8", mutates_args=(), device_types="cuda")
def linear_i8(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
              bias: Optional[torch.Tensor]) -> torch.Tensor:
    """int8 [M,Kp] x int8 [N,Kp]^T with the fused per-token / per-channel scale, bias and bf16 cast."""
    return _linear(xq, sx, wq, sw, bias, False, False)[0]


@torch.library.custom_op("daxq::linear_i8_acc", mutates_args=(), device_types="cuda")
def linear_i8_acc(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                  bias: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
    """As linear_i8, also returning the exact int32 accumulators [M,N]."""
    return _linear(xq, sx, wq, sw, bias, False, True)


@torch.library.custom_op("daxq::linear_e4m3", mutates_args=(), device_types="cuda")
def linear_e4m3(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                bias: Optional[torch.Tensor]) -> torch.Tensor:
    """e4m3fn [M,Kp] x e4m3fn [N,Kp]^T (bytes as uint8), fp32 accumulate, fused scales + bias + bf16."""
    return _linear(xq, sx, wq, sw, bias, True, False)[0]


@torch.library.custom_op("daxq::linear_e4m3_acc", mutates_args=(), device_types="cuda")
def linear_e4m3_acc(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                    bias: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
    return _linear(xq, sx, wq, sw, bias, True, True)


@torch.library.custom_op("daxq::linear_e5m2_e4m3", mutates_args=(), device_types="cuda")
def linear_e5m2_e4m3(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                     bias: Optional[torch.Tensor]) -> torch.Tensor:
    """e5m2 activation bytes [M,Kp] x e4m3fn weight bytes [N,Kp]^T, fp32 accumulate, fused epilogue."""
    return _linear(xq, sx, wq, sw, bias, True, False, True)[0]


@torch.library.custom_op("daxq::linear_e5m2_e4m3_acc", mutates_args=(), device_types="cuda")
def linear_e5m2_e4m3_acc(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor,
                         bias: Optional[torch.Tensor]) -> Tuple[torch.Tensor, torch.Tensor]:
    return _linear(xq, sx, wq, sw, bias, True, True, True)


def _lin_fake(xq, sx, wq, sw, bias):
    return xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16)


linear_i8.register_fake(_lin_fake)
linear_e4m3.register_fake(_lin_fake)
linear_e5m2_e4m3.register_fake(_lin_fake)
linear_e5m2_e4m3_acc.register_fake(lambda xq, sx, wq, sw, bias: (
    _lin_fake(xq, sx, wq, sw, bias), xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.float32)))
linear_i8_acc.register_fake(lambda xq, sx, wq, sw, bias: (
    _lin_fake(xq, sx, wq, sw, bias), xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.int32)))
linear_e4m3_acc.register_fake(lambda xq, sx, wq, sw, bias: (
    _lin_fake(xq, sx, wq, sw, bias), xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.float32)))


# ----------------------------------------------------------------------------- quantiser + GEMM behind one dispatch
def _dynamic_linear(x, wq, sw, bias, fmt: str):
    """Per-token quantiser and GEMM of one linear, the same two launches as act_quant_* + linear_*; one op call
    instead of two halves the host time per forward, which is what a small linear costs."""
    fp8 = fmt != "i8"
    _same_device("dynamic_linear_" + fmt, x, wq=wq, sw=sw, bias=bias)  # before the quantiser is launched
    xq, sx = _act_quant(x, fp8, fmt == "e5m2")
    if xq.shape[1] != wq.shape[1]:
        raise ValueError(f"daxq::dynamic_linear_{fmt}: x has K={x.shape[1]} (padded {xq.shape[1]}), the weight {wq.shape[1]}")
    return _linear(xq, sx, wq, sw, bias, fp8, False, fmt == "e5m2")[0]


@torch.library.custom_op("daxq::dynamic_linear_i8", mutates_args=(), device_types="cuda")
def dynamic_linear_i8(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """bf16 [M,K] -> per-token int8 -> x int8 [N, pad128(K)]^T with the fused epilogue -> bf16 [M,N]."""
    return _dynamic_linear(x, wq, sw, bias, "i8")


@torch.library.custom_op("daxq::dynamic_linear_e4m3", mutates_args=(), device_types="cuda")
def dynamic_linear_e4m3(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    return _dynamic_linear(x, wq, sw, bias, "e4m3")


@torch.library.custom_op("daxq::dynamic_linear_e5m2_e4m3", mutates_args=(), device_types="cuda")
def dynamic_linear_e5m2_e4m3(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    return _dynamic_linear(x, wq, sw, bias, "e5m2")


def _dyn_fake(x, wq, sw, bias):
    return x.new_empty((x.shape[0], wq.shape[0]), dtype=torch.bfloat16)


dynamic_linear_i8.register_fake(_dyn_fake)
dynamic_linear_e4m3.register_fake(_dyn_fake)
dynamic_linear_e5m2_e4m3.register_fake(_dyn_fake)


# ----------------------------------------------------------------------------- per-tensor scales
@torch.library.custom_op("daxq::tensor_scale", mutates_args=(), device_types="cuda")
def tensor_scale(row_min: torch.Tensor, row_max: torch.Tensor, qmax: float, round_bf16: bool,
                 n_expand: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-tensor scale from per-row (min, max): (scale fp32 [1], the same value n_expand times)."""
    _need_gpu(row_min, "tensor_scale")
    _same_device("tensor_scale", row_min, row_max=row_max)
    if row_min.dtype != torch.float32 or row_max.dtype != torch.float32 or row_min.shape != row_max.shape or row_min.numel() == 0:
        raise ValueError("daxq::tensor_scale: row_min / row_max must be non-empty fp32 tensors of one shape")
    lo, hi = row_min.contiguous(), row_max.contiguous()
    with _on_device(lo):
        s1 = torch.empty((1,), dtype=torch.float32, device=lo.device)
        ex = torch.empty((n_expand,), dtype=torch.float32, device=lo.device)
        _capi.check(_capi.lib().daxq_tensor_scale(lo.data_ptr(), hi.data_ptr(), lo.numel(), float(qmax), int(round_bf16),
                                                  s1.data_ptr(), ex.data_ptr() if n_expand else 0, n_expand, _stream(lo)),
                    "tensor_scale")
    return s1, ex


tensor_scale.register_fake(lambda row_min, row_max, qmax, round_bf16, n_expand: (
    row_min.new_empty((1,), dtype=torch.float32), row_min.new_empty((n_expand,), dtype=torch.float32)))


@torch.library.custom_op("daxq::tensor_minmax_update", mutates_args=("min_inout", "max_inout"), device_types="cuda")
def tensor_minmax_update(row_min: torch.Tensor, row_max: torch.Tensor, min_inout: torch.Tensor,
                         max_inout: torch.Tensor) -> None:
    """min_inout[0] = min(min_inout[0], min(row_min)); max_inout likewise (fp32, one element each)."""
    _need_gpu(row_min, "tensor_minmax_update")
    for t in (row_min, row_max, min_inout, max_inout):
        if t.dtype != torch.float32 or t.device != row_min.device or not t.is_contiguous():
            raise ValueError("daxq::tensor_minmax_update: contiguous fp32 tensors on one device expected")
    if min_inout.numel() != 1 or max_inout.numel() != 1 or row_min.numel() == 0 or row_min.numel() != row_max.numel():
        raise ValueError("daxq::tensor_minmax_update: bad shapes")
    with _on_device(row_min):
        _capi.check(_capi.lib().daxq_tensor_minmax_update(row_min.data_ptr(), row_max.data_ptr(), row_min.numel(),
                                                          min_inout.data_ptr(), max_inout.data_ptr(), _stream(row_min)),
                    "tensor_minmax_update")


tensor_minmax_update.register_fake(lambda row_min, row_max, min_inout, max_inout: None)


@torch.library.custom_op("daxq::broadcast_f32", mutates_args=(), device_types="cuda")
def broadcast_f32(src: torch.Tensor, n: int) -> torch.Tensor:
    """fp32 [n] filled with src[0] (a stored per-tensor scale as the vector the kernels take)."""
    _need_gpu(src, "broadcast_f32")
    if src.dtype != torch.float32 or src.numel() != 1:
        raise ValueError("daxq::broadcast_f32: src must hold one fp32 value")
    with _on_device(src):
        dst = torch.empty((n,), dtype=torch.float32, device=src.device)
        _capi.check(_capi.lib().daxq_broadcast_f32(src.data_ptr(), dst.data_ptr(), n, _stream(src)), "broadcast_f32")
    return dst


broadcast_f32.register_fake(lambda src, n: src.new_empty((n,), dtype=torch.float32))

