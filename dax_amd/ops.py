"""``torch.ops.daxq.*``: the HIP kernels of libdaxq as PyTorch custom ops.

Each op allocates its outputs with torch (device memory is torch's), passes raw device
pointers and the current HIP stream through the C ABI, and has a fake (meta) kernel so a
surrounding ``torch.compile`` graph can trace through it.  No op has a CPU kernel.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

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


_multi_gpu = None


def _on_device(t: torch.Tensor):
    """Context that makes the tensor's device current for the allocations and the launch; with a single GPU it is
    current already and the guard (several microseconds per call) is left out."""
    global _multi_gpu
    if _multi_gpu is None:
        _multi_gpu = torch.cuda.device_count() > 1
    return torch.cuda.device(t.device) if _multi_gpu else _NO_GUARD


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


FLOAT_KIND = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}  # DAXQ_BF16 / DAXQ_F16 / DAXQ_F32
FMT = {"i8": 0, "e4m3": 1, "e5m2": 2}  # DAXQ_FMT_*
FMT_OF_DTYPE = {torch.int8: "i8", torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}
QMAX = {"i8": 127.0, "e4m3": 448.0, "e5m2": 57344.0}
EPS_F32 = 1.1920928955078125e-07  # torch.finfo(torch.float32).eps = 2^-23, the floor the reference's wrappers pass


def _rows_float(x: torch.Tensor, what: str) -> int:
    """Checks a [rows, K] matrix of one of the element types the reference's quantisers accept
    (dax/quant/nn/dynamic/functional.py:99-103) and returns its DAXQ_* type code."""
    _need_gpu(x, what)
    if x.dtype not in FLOAT_KIND:
        raise AssertionError(f"Unsupported input dtype: {x.dtype}")
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError(f"daxq::{what}: expected a 2-d tensor with contiguous rows, got shape {tuple(x.shape)} "
                         f"strides {x.stride()}")
    return FLOAT_KIND[x.dtype]


def _rows_bf16(x: torch.Tensor, what: str) -> None:
    _need_gpu(x, what)
    if x.dtype != torch.bfloat16:
        raise NotImplementedError(f"daxq::{what}: only bfloat16 inputs are implemented, got {x.dtype}")
    if x.dim() != 2 or x.stride(1) != 1:
        raise ValueError(f"daxq::{what}: expected a 2-d tensor with contiguous rows, got shape {tuple(x.shape)} "
                         f"strides {x.stride()}")


# ----------------------------------------------------------------------------- act quant
# Rows of a quantised activation whose length is a multiple of 1 KB are kept 128 bytes further apart than they are
# long.  The GEMM streams 256-row panels, every row at the same K offset; with a row stride that is a multiple of 1 KB
# (K = 5120: 40 lines of 128 bytes) those addresses fall onto few memory channels, an odd number of lines per row
# spreads them.  Measured on the 14B shapes inside the benchmark step: +0.4 to +2 % on the K = 5120 launches (INT8 GEMM
# average +0.55 %), nothing or a small loss at K = 13824, which keeps its rows contiguous.  The pad is never read or
# written.
Q_ROW_PAD = 128
MIN_TILE_ROWS = 128  # rows of the smallest tile of the tiled GEMM kernels


def _row_pad(kp: int) -> int:
    return Q_ROW_PAD if kp % 1024 == 0 else 0


def _alloc_q(m: int, kp: int, dtype, device) -> torch.Tensor:
    pad = _row_pad(kp)
    q = torch.empty((m, kp + pad), dtype=dtype, device=device)
    return q[:, :kp] if pad else q


def _fake_q(x, m: int, kp: int, dtype) -> torch.Tensor:
    return x.new_empty_strided((m, kp), (kp + _row_pad(kp), 1), dtype=dtype)


def _act_quant(x: torch.Tensor, fp8, e5m2: bool = False, rows: int = 0, scale_fp32: bool = False,
               quant_max: float = 0.0, eps: float = -1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """rows > M: the buffers get that many rows and only the first M are written.  scale_fp32: the scale is not rounded
    to x's element type.  quant_max <= 0 / eps < 0: the format's own maximum / 2^-23."""
    fmt = "e5m2" if e5m2 else "e4m3" if fp8 else "i8"
    name = "act_quant_" + fmt
    kind = _rows_float(x, name)
    m, k = x.shape
    kp = pad_k(k)
    with _on_device(x):
        q = _alloc_q(max(m, rows), kp, torch.uint8 if fp8 else torch.int8, x.device)
        s = torch.empty((max(m, rows),), dtype=torch.float32, device=x.device)
        if m:
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(_capi.lib().daxq_act_quant_rows_ex(
                x.data_ptr(), kind, FMT[fmt], m, k, ld_x, q.data_ptr(), kp + _row_pad(kp), s.data_ptr(),
                quant_max if quant_max > 0 else QMAX[fmt], eps if eps >= 0 else EPS_F32, 0 if scale_fp32 else 1, _stream(x)), name)
    return q, s


@torch.library.custom_op("daxq::act_quant_i8", mutates_args=(), device_types="cuda")
def act_quant_i8(x: torch.Tensor, scale_fp32: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 / fp16 / fp32 [M,K] -> (int8 [M, pad128(K)] zero padded, fp32 [M] per-token scale).  scale_fp32: the scale
    stays in fp32 instead of being rounded to x's element type (the reference's forward under its torch.compile decorator)."""
    return _act_quant(x, False, scale_fp32=scale_fp32)


@torch.library.custom_op("daxq::act_quant_e4m3", mutates_args=(), device_types="cuda")
def act_quant_e4m3(x: torch.Tensor, scale_fp32: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [M,K] -> (e4m3fn bytes as uint8 [M, pad128(K)], fp32 [M] per-token scale)."""
    return _act_quant(x, True, scale_fp32=scale_fp32)


@torch.library.custom_op("daxq::act_quant_e5m2", mutates_args=(), device_types="cuda")
def act_quant_e5m2(x: torch.Tensor, scale_fp32: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """bf16 [M,K] -> (e5m2 bytes as uint8 [M, pad128(K)], fp32 [M] per-token scale)."""
    return _act_quant(x, True, True, scale_fp32=scale_fp32)


@torch.library.custom_op("daxq::act_quant_rows", mutates_args=(), device_types="cuda")
def act_quant_rows(x: torch.Tensor, fmt: str, quant_max: float, eps: float, round_scale: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """The per-row quantiser with the caller's quant_max and eps (dax/quant/nn/dynamic/functional.py:54-61): fmt "i8" /
    "e4m3" / "e5m2"; round_scale: quotient and floor are rounded to x's element type (the eager chain) or stay fp32."""
    if fmt not in FMT:
        raise ValueError(f"daxq::act_quant_rows: unknown format {fmt}")
    if not quant_max > 0 or not eps >= 0:
        raise ValueError("daxq::act_quant_rows: quant_max must be positive and eps not negative")
    return _act_quant(x, fmt != "i8", fmt == "e5m2", scale_fp32=not round_scale, quant_max=quant_max, eps=eps)


def _act_quant_fake(x, dtype):
    return _fake_q(x, x.shape[0], pad_k(x.shape[1]), dtype), x.new_empty((x.shape[0],), dtype=torch.float32)


act_quant_i8.register_fake(lambda x, scale_fp32=False: _act_quant_fake(x, torch.int8))
act_quant_e4m3.register_fake(lambda x, scale_fp32=False: _act_quant_fake(x, torch.uint8))
act_quant_e5m2.register_fake(lambda x, scale_fp32=False: _act_quant_fake(x, torch.uint8))
act_quant_rows.register_fake(lambda x, fmt, quant_max, eps, round_scale: _act_quant_fake(x, torch.int8 if fmt == "i8" else torch.uint8))


# ----------------------------------------------------------------------------- producer + act quant
_FMT_NAMES = ("i8", "e4m3", "e5m2")


def _fused_out(x: torch.Tensor, fmt: str, want_y: bool):
    m, k = x.shape
    q = _alloc_q(m, pad_k(k), torch.int8 if fmt == "i8" else torch.uint8, x.device)
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
                           rows_per_group, eps, y.data_ptr() if want_y else 0, k, q.data_ptr(), q.stride(0),
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
            _capi.check(fn(x.data_ptr(), m, k, ld_x, y.data_ptr() if want_y else 0, k, q.data_ptr(), q.stride(0),
                           s.data_ptr(), _stream(x)), name)
    return q, s, y


def _fused_fake(x, fmt, want_y):
    return (_fake_q(x, x.shape[0], pad_k(x.shape[1]), torch.int8 if fmt == "i8" else torch.uint8),
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
    kind = _rows_float(x, name)
    m, k = x.shape
    if scale.dtype != torch.float32 or scale.numel() != m or scale.device != x.device:
        raise ValueError(f"daxq::{name}: scale must be fp32 with one value per row on {x.device}")
    scale = scale.reshape(-1).contiguous()
    ld_q = pad_k(k) if padded else k
    with _on_device(x):
        q = torch.empty((m, ld_q), dtype=torch.int8 if fmt == "i8" else torch.uint8, device=x.device)
        if m:
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(_capi.lib().daxq_quantize_rows(x.data_ptr(), kind, FMT[fmt], m, k, ld_x, scale.data_ptr(),
                                                       q.data_ptr(), ld_q, _stream(x)), name)
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
    """Per-row (min, max) of a bf16 / fp16 / fp32 matrix in fp32."""
    kind = _rows_float(x, "row_minmax")
    m, k = x.shape
    with _on_device(x):
        lo = torch.empty((m,), dtype=torch.float32, device=x.device)
        hi = torch.empty((m,), dtype=torch.float32, device=x.device)
        if m:
            ld_x = x.stride(0) if m > 1 else k
            _capi.check(_capi.lib().daxq_row_minmax_t(x.data_ptr(), kind, m, k, ld_x, lo.data_ptr(), hi.data_ptr(),
                                                      _stream(x)), "row_minmax")
    return lo, hi


row_minmax.register_fake(lambda x: (x.new_empty((x.shape[0],), dtype=torch.float32),
                                    x.new_empty((x.shape[0],), dtype=torch.float32)))


@torch.library.custom_op("daxq::scale_from_minmax", mutates_args=(), device_types="cuda")
def scale_from_minmax(min_val: torch.Tensor, max_val: torch.Tensor, qmax: float, eps: float = EPS_F32) -> torch.Tensor:
    """max(max(-min, max) / qmax, eps) element-wise in fp32."""
    _need_gpu(min_val, "scale_from_minmax")
    _same_device("scale_from_minmax", min_val, max_val=max_val)
    if min_val.dtype != torch.float32 or max_val.dtype != torch.float32 or min_val.shape != max_val.shape:
        raise ValueError("daxq::scale_from_minmax: min/max must be fp32 tensors of one shape")
    lo, hi = min_val.contiguous(), max_val.contiguous()
    with _on_device(lo):
        s = torch.empty_like(lo)
        _capi.check(_capi.lib().daxq_scale_from_minmax_eps(lo.data_ptr(), hi.data_ptr(), lo.numel(), float(qmax), float(eps),
                                                           s.data_ptr(), _stream(lo)), "scale_from_minmax")
    return s


scale_from_minmax.register_fake(lambda min_val, max_val, qmax, eps=EPS_F32: torch.empty_like(min_val))


# ----------------------------------------------------------------------------- GEMM + epilogue
# Workspaces of the split-K launches: one per (device, stream), zero-filled when it is made (the kernels leave the
# counters at its head zero).  Launches on one stream are ordered, so they can share it; another stream gets its own.
# A workspace is never freed once a launch has used it: its address may sit in work that is still queued.  The first
# one of a stream already holds everything the library's own choice of ranges can ask for (tiles x ranges <= 256); a
# larger explicit request gets a larger one and the old one stays alive beside it.
_splitk_ws = {}
_splitk_retired = []  # outgrown workspaces, kept alive until the process ends
SPLITK_AUTO = True  # few-tile launches (a few hundred rows) cut K into ranges when it pays
SPLITK_WS_BYTES = 16384 + 256 * 65536  # counters + 256 partial results of 64 KiB


def _splitk_workspace(device, stream: int, need: int):
    """None while the stream is being captured: a graph replays on whatever stream its owner picks, possibly beside
    another graph captured on the same stream, and two replays that share one workspace race on its counters.  The
    caller then takes the plain launch (INT8 results are the same bits either way)."""
    if torch.cuda.is_current_stream_capturing():
        return None
    key = (device.index, stream)
    ws = _splitk_ws.get(key)
    if ws is None or ws.numel() < need:
        if ws is not None:
            _splitk_retired.append(ws)
        ws = torch.zeros(max(need, SPLITK_WS_BYTES), dtype=torch.uint8, device=device)
        _splitk_ws[key] = ws
    return ws


def _auto_splits(m: int, n: int, k: int, out_dtype, want_acc: bool, fp8: bool) -> int:
    # INT8 only: its partial sums are integers, so the result does not depend on how K is cut and a row's output stays
    # the same whatever the batch it arrives in; FP8 sums would change in the last bits with the number of rows
    if not SPLITK_AUTO or fp8 or want_acc or out_dtype != torch.bfloat16 or _capi.kernel_arg() != 0:
        return 1
    return _capi.lib().daxq_linear_splitk_choice(m, n, k)


def _linear(xq, sx, wq, sw, bias, fp8: bool, want_acc: bool, x_e5m2: bool = False, w_e5m2: bool = False,
            out_dtype: torch.dtype = torch.bfloat16, splits: Optional[int] = None):
    x_fmt = "e5m2" if x_e5m2 else "e4m3" if fp8 else "i8"
    w_fmt = "e5m2" if w_e5m2 else "e4m3" if fp8 else "i8"
    name = f"linear_{x_fmt}_{w_fmt}"
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
    if out_dtype not in FLOAT_KIND:
        raise ValueError(f"daxq::{name}: out_dtype must be bfloat16, float16 or float32, got {out_dtype}")
    if bias is not None and (bias.dtype != out_dtype or bias.numel() != n):
        raise ValueError(f"daxq::{name}: bias must be {out_dtype} [N]")
    sx = sx.reshape(-1).contiguous()
    sw = sw.reshape(-1).contiguous()
    bias_c = bias.contiguous() if bias is not None else None
    with _on_device(xq):
        out = torch.empty((m, n), dtype=out_dtype, device=xq.device)
        acc = torch.empty((m, n), dtype=torch.float32 if fp8 else torch.int32, device=xq.device) if want_acc else None
        if m and n:
            ld_x = xq.stride(0) if m > 1 else k
            ld_w = wq.stride(0) if n > 1 else k
            splits = splits if splits is not None else _auto_splits(m, n, k, out_dtype, want_acc, fp8)
            if splits > 1:
                stream = _stream(xq)
                need = _capi.lib().daxq_linear_splitk_workspace_bytes(m, n, splits)
                ws = _splitk_workspace(xq.device, stream, need)
                if ws is not None:
                    _capi.check(_capi.lib().daxq_linear_w8a8_splitk(
                        FMT[x_fmt], FMT[w_fmt], xq.data_ptr(), ld_x, sx.data_ptr(), wq.data_ptr(), ld_w, sw.data_ptr(),
                        bias_c.data_ptr() if bias_c is not None else None, out.data_ptr(), n, m, n, k, splits,
                        ws.data_ptr(), ws.numel(), stream), name + "_splitk")
                    return out, acc
            _capi.check(_capi.lib().daxq_linear_w8a8(
                FMT[x_fmt], FMT[w_fmt], FLOAT_KIND[out_dtype], xq.data_ptr(), ld_x, sx.data_ptr(), wq.data_ptr(), ld_w,
                sw.data_ptr(), bias_c.data_ptr() if bias_c is not None else None, out.data_ptr(), n,
                acc.data_ptr() if acc is not None else None, n, m, n, k, _capi.kernel_arg(), _stream(xq)), name)
    return out, acc


@torch.library.custom_op("daxq::linear_w8a8", mutates_args=(), device_types="cuda")
def linear_w8a8(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                x_fmt: str, w_fmt: str, out_dtype: torch.dtype) -> torch.Tensor:
    """The GEMM + epilogue for any operand pairing ("i8" x "i8", or "e4m3" / "e5m2" activations against "e4m3" /
    "e5m2" weights, bytes as uint8) and any module dtype: out and bias are bf16, fp16 or fp32."""
    if (x_fmt == "i8") != (w_fmt == "i8") or x_fmt not in FMT or w_fmt not in FMT:
        raise ValueError(f"daxq::linear_w8a8: unsupported operand formats {x_fmt} x {w_fmt}")
    return _linear(xq, sx, wq, sw, bias, x_fmt != "i8", False, x_fmt == "e5m2", w_fmt == "e5m2", out_dtype)[0]


@torch.library.custom_op("daxq::linear_w8a8_acc", mutates_args=(), device_types="cuda")
def linear_w8a8_acc(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                    x_fmt: str, w_fmt: str, out_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """As linear_w8a8, also returning the raw accumulators (int32 / fp32 [M,N])."""
    if (x_fmt == "i8") != (w_fmt == "i8") or x_fmt not in FMT or w_fmt not in FMT:
        raise ValueError(f"daxq::linear_w8a8: unsupported operand formats {x_fmt} x {w_fmt}")
    return _linear(xq, sx, wq, sw, bias, x_fmt != "i8", True, x_fmt == "e5m2", w_fmt == "e5m2", out_dtype)


@torch.library.custom_op("daxq::linear_w8a8_splitk", mutates_args=(), device_types="cuda")
def linear_w8a8_splitk(xq: torch.Tensor, sx: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                       x_fmt: str, w_fmt: str, splits: int) -> torch.Tensor:
    """linear_w8a8 (bf16) with K cut into `splits` ranges that run as separate workgroups (0 = the library's choice):
    for launches with too few output tiles to fill the device."""
    if (x_fmt == "i8") != (w_fmt == "i8") or x_fmt not in FMT or w_fmt not in FMT:
        raise ValueError(f"daxq::linear_w8a8_splitk: unsupported operand formats {x_fmt} x {w_fmt}")
    if splits == 0:
        splits = _capi.lib().daxq_linear_splitk_choice(xq.shape[0], wq.shape[0], xq.shape[1])
    return _linear(xq, sx, wq, sw, bias, x_fmt != "i8", False, x_fmt == "e5m2", w_fmt == "e5m2", torch.bfloat16, splits)[0]


linear_w8a8_splitk.register_fake(lambda xq, sx, wq, sw, bias, x_fmt, w_fmt, splits:
                                 xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.bfloat16))
linear_w8a8.register_fake(lambda xq, sx, wq, sw, bias, x_fmt, w_fmt, out_dtype:
                          xq.new_empty((xq.shape[0], wq.shape[0]), dtype=out_dtype))
linear_w8a8_acc.register_fake(lambda xq, sx, wq, sw, bias, x_fmt, w_fmt, out_dtype: (
    xq.new_empty((xq.shape[0], wq.shape[0]), dtype=out_dtype),
    xq.new_empty((xq.shape[0], wq.shape[0]), dtype=torch.int32 if x_fmt == "i8" else torch.float32)))


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
_Q_DTYPE = {"i8": torch.int8, "e4m3": torch.uint8, "e5m2": torch.uint8}
_W_FMT = {"i8": 0, "e4m3": 1, "e5m2": 1}  # the weight format each activation format is paired with here
_splitk_memo = {}  # (rows, n, kp) -> daxq_linear_splitk_choice, host arithmetic asked once per shape
_dyn_fn = None     # the bound daxq_dynamic_linear


def _dynamic_linear(x, wq, sw, bias, fmt: str, scale_fp32: bool = False):
    """Per-token quantiser and GEMM of one linear through the library's single entry point for the pair
    (daxq_dynamic_linear): one ctypes call, and two allocations (the quantised activation with its scales behind it
    in one buffer, and the output) behind one op dispatch -- the host time per forward is what a small linear costs.
    The launches are those of act_quant_* followed by linear_*."""
    global _dyn_fn
    dev = x.device
    kind = FLOAT_KIND.get(x.dtype)
    if dev.type != "cuda" or kind is None or x.dim() != 2 or x.stride(1) != 1:
        _rows_float(x, "dynamic_linear_" + fmt)  # raises with the reason
    if dev.index not in _capi._checked_devices:
        _need_gpu(x, "dynamic_linear_" + fmt)
    if wq.device != dev or sw.device != dev or (bias is not None and bias.device != dev):
        _same_device("dynamic_linear_" + fmt, x, wq=wq, sw=sw, bias=bias)  # before anything is launched
    if wq.dtype != _Q_DTYPE[fmt] or wq.dim() != 2 or wq.stride(1) != 1:
        raise ValueError(f"daxq::dynamic_linear_{fmt}: the weight must be {_Q_DTYPE[fmt]} [N, pad128(K)] with contiguous rows")
    m, k = x.shape
    n, kp = wq.shape
    if kp != (k + K_ALIGN - 1) // K_ALIGN * K_ALIGN:
        raise ValueError(f"daxq::dynamic_linear_{fmt}: x has K={k} (padded {pad_k(k)}), the weight {kp}")
    if sw.dtype != torch.float32 or sw.numel() != n or not sw.is_contiguous():
        raise ValueError(f"daxq::dynamic_linear_{fmt}: sw must be contiguous fp32 [N]")
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != n or not bias.is_contiguous()):
        raise ValueError(f"daxq::dynamic_linear_{fmt}: bias must be contiguous bfloat16 [N]")
    # Fewer rows than one 128-row tile: the buffers get 128 rows and the tiled kernel runs on all of them (twice as fast
    # as the kernel that takes fewer rows); what the rows beyond M hold is never looked at, and their outputs are cut off.
    rows = MIN_TILE_ROWS if 0 < m < MIN_TILE_ROWS <= n else m
    ld_q = kp + (Q_ROW_PAD if kp % 1024 == 0 else 0)
    with _on_device(x):
        # quantised rows, then the fp32 scales (the row stride is a multiple of 128, so they are aligned)
        scratch = torch.empty((rows * (ld_q + 4),), dtype=torch.uint8, device=dev)
        out = torch.empty((rows, n), dtype=torch.bfloat16, device=dev)
        if m and n:
            if _dyn_fn is None:
                _dyn_fn = _capi.lib().daxq_dynamic_linear
            stream = _stream(x)
            ws_ptr, ws_bytes = None, 0
            karg = _capi.kernel_arg()
            if fmt == "i8" and SPLITK_AUTO and karg == 0:
                key = (rows, n, kp)
                splits = _splitk_memo.get(key)
                if splits is None:
                    splits = _splitk_memo[key] = _capi.lib().daxq_linear_splitk_choice(rows, n, kp)
                if splits > 1:
                    ws = _splitk_workspace(dev, stream, SPLITK_WS_BYTES)
                    if ws is not None:
                        ws_ptr, ws_bytes = ws.data_ptr(), ws.numel()
            base = scratch.data_ptr()
            rc = _dyn_fn(kind, FMT[fmt], _W_FMT[fmt], 0, 0 if scale_fp32 else 1, x.data_ptr(), x.stride(0) if m > 1 else k, base, ld_q,
                         base + rows * ld_q, rows, wq.data_ptr(), wq.stride(0) if n > 1 else kp, sw.data_ptr(),
                         bias.data_ptr() if bias is not None else None, out.data_ptr(), n, m, n, k, ws_ptr, ws_bytes, karg,
                         stream)
            if rc:
                _capi.check(rc, "dynamic_linear_" + fmt)
    return out[:m] if rows != m else out


@torch.library.custom_op("daxq::dynamic_linear_i8", mutates_args=(), device_types="cuda")
def dynamic_linear_i8(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                        scale_fp32: bool = False) -> torch.Tensor:
    """bf16 [M,K] -> per-token int8 -> x int8 [N, pad128(K)]^T with the fused epilogue -> bf16 [M,N]."""
    return _dynamic_linear(x, wq, sw, bias, "i8", scale_fp32)


@torch.library.custom_op("daxq::dynamic_linear_e4m3", mutates_args=(), device_types="cuda")
def dynamic_linear_e4m3(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                          scale_fp32: bool = False) -> torch.Tensor:
    return _dynamic_linear(x, wq, sw, bias, "e4m3", scale_fp32)


@torch.library.custom_op("daxq::dynamic_linear_e5m2_e4m3", mutates_args=(), device_types="cuda")
def dynamic_linear_e5m2_e4m3(x: torch.Tensor, wq: torch.Tensor, sw: torch.Tensor, bias: Optional[torch.Tensor],
                               scale_fp32: bool = False) -> torch.Tensor:
    return _dynamic_linear(x, wq, sw, bias, "e5m2", scale_fp32)


def _dyn_fake(x, wq, sw, bias, scale_fp32=False):
    return x.new_empty((x.shape[0], wq.shape[0]), dtype=torch.bfloat16)


dynamic_linear_i8.register_fake(_dyn_fake)
dynamic_linear_e4m3.register_fake(_dyn_fake)
dynamic_linear_e5m2_e4m3.register_fake(_dyn_fake)


# ----------------------------------------------------------------------------- per-tensor scales
@torch.library.custom_op("daxq::tensor_scale", mutates_args=(), device_types="cuda")
def tensor_scale(row_min: torch.Tensor, row_max: torch.Tensor, qmax: float, round_bf16: int,
                 n_expand: int, eps: float = EPS_F32) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-tensor scale from per-row (min, max): (scale fp32 [1], the same value n_expand times).  round_bf16: the
    quotient is rounded to bf16 (1) or fp16 (2), the element type of the tensor the statistics come from, or not
    at all (0: fp32 tensors and the observer rule)."""
    _need_gpu(row_min, "tensor_scale")
    _same_device("tensor_scale", row_min, row_max=row_max)
    if row_min.dtype != torch.float32 or row_max.dtype != torch.float32 or row_min.shape != row_max.shape or row_min.numel() == 0:
        raise ValueError("daxq::tensor_scale: row_min / row_max must be non-empty fp32 tensors of one shape")
    lo, hi = row_min.contiguous(), row_max.contiguous()
    with _on_device(lo):
        s1 = torch.empty((1,), dtype=torch.float32, device=lo.device)
        ex = torch.empty((n_expand,), dtype=torch.float32, device=lo.device)
        _capi.check(_capi.lib().daxq_tensor_scale(lo.data_ptr(), hi.data_ptr(), lo.numel(), float(qmax), float(eps), int(round_bf16),
                                                  s1.data_ptr(), ex.data_ptr() if n_expand else 0, n_expand, _stream(lo)),
                    "tensor_scale")
    return s1, ex


tensor_scale.register_fake(lambda row_min, row_max, qmax, round_bf16, n_expand, eps=EPS_F32: (
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




# ----------------------------------------------------------------------------- any block shape
def _view_args(view_shape, reduced):
    import ctypes as C

    nd = len(view_shape)
    if nd != len(reduced) or not 1 <= nd <= 8:
        raise NotImplementedError(f"daxq block kernels take views of 1 to 8 dimensions, got {nd}")
    return nd, (C.c_int64 * nd)(*[int(v) for v in view_shape]), (C.c_int32 * nd)(*[int(bool(r)) for r in reduced])


@torch.library.custom_op("daxq::block_scale", mutates_args=(), device_types="cuda")
def block_scale(x: torch.Tensor, view_shape: List[int], reduced: List[int], qmax: float, round_to_x: bool,
                eps: float = EPS_F32) -> torch.Tensor:
    """Scale of every block of the contiguous tensor x seen through `view_shape`, a block spanning the dimensions
    flagged in `reduced`: fp32, one element per kept index (row-major over the kept dimensions)."""
    _need_gpu(x, "block_scale")
    if x.dtype not in FLOAT_KIND:
        raise AssertionError(f"Unsupported input dtype: {x.dtype}")
    if not x.is_contiguous():
        raise ValueError("daxq::block_scale: x must be contiguous")
    nd, vs, rd = _view_args(view_shape, reduced)
    kept = 1
    total = 1
    for v, r in zip(view_shape, reduced):
        total *= v
        kept *= 1 if r else v
    if total != x.numel():
        raise ValueError(f"daxq::block_scale: view {list(view_shape)} does not hold {x.numel()} elements")
    with _on_device(x):
        s = torch.empty((kept,), dtype=torch.float32, device=x.device)
        if total:
            _capi.check(_capi.lib().daxq_block_scale(x.data_ptr(), FLOAT_KIND[x.dtype], nd, vs, rd, float(qmax), float(eps),
                                                     int(round_to_x), s.data_ptr(), _stream(x)), "block_scale")
    return s


@torch.library.custom_op("daxq::block_quantize", mutates_args=(), device_types="cuda")
def block_quantize(x: torch.Tensor, view_shape: List[int], reduced: List[int], scale: torch.Tensor, fmt: str,
                   scale_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Leaf quantiser of every element of x with its block's scale (the output of block_scale): int8, or fp8 bytes as
    uint8, in x's shape.  scale_dtype: the type of the scale the caller asked for, which decides the type the arithmetic
    runs in (type promotion of x and the scale); the values are passed as fp32."""
    _need_gpu(x, "block_quantize")
    _same_device("block_quantize", x, scale=scale)
    if x.dtype not in FLOAT_KIND or fmt not in FMT:
        raise AssertionError(f"Unsupported input dtype / format: {x.dtype} / {fmt}")
    if not x.is_contiguous() or scale.dtype != torch.float32 or not scale.is_contiguous():
        raise ValueError("daxq::block_quantize: x and scale must be contiguous, scale fp32")
    nd, vs, rd = _view_args(view_shape, reduced)
    kept = 1
    for v, r in zip(view_shape, reduced):
        kept *= 1 if r else v
    if kept != scale.numel():
        raise ValueError(f"daxq::block_quantize: {scale.numel()} scales for {kept} blocks")
    with _on_device(x):
        q = torch.empty(x.shape, dtype=torch.int8 if fmt == "i8" else torch.uint8, device=x.device)
        if x.numel():
            _capi.check(_capi.lib().daxq_block_quantize(x.data_ptr(), FLOAT_KIND[x.dtype], FMT[fmt], nd, vs, rd,
                                                        scale.data_ptr(), FLOAT_KIND[scale_dtype], q.data_ptr(), _stream(x)),
                        "block_quantize")
    return q


def _block_scale_fake(x, view_shape, reduced, qmax, round_to_x, eps=EPS_F32):
    kept = 1
    for v, r in zip(view_shape, reduced):
        kept *= 1 if r else v
    return x.new_empty((kept,), dtype=torch.float32)


block_scale.register_fake(_block_scale_fake)
block_quantize.register_fake(lambda x, view_shape, reduced, scale, fmt, scale_dtype=torch.float32: x.new_empty(x.shape, dtype=torch.int8 if fmt == "i8" else torch.uint8))
