"""Leaf quantisers: a tensor and the scale of each of its rows in, quantised values out.

Same names and argument meaning as dax/quant/nn/quantized/functional.py:4-20; the work is
done by the HIP kernels ``daxq_quantize_rows_*`` (int8: reciprocal-multiply, round half to
even, clamp; e4m3fn / e5m2: true division, clamp to +-448 / +-57344, round to nearest even).
A scale of one element (per-tensor scheme) is written out as one value per row on the device.
"""
import torch
from torch import Tensor

from .... import ops

FP8_ALLOWED_DTYPES = (
    torch.float8_e4m3fn,
    torch.float8_e5m2,
)


def _rows_and_scale(x: Tensor, scale: Tensor):
    """Flattens x to [rows, K] and gives every row its scale (scale broadcasts against x
    with a trailing dimension of 1, or is a single value)."""
    k = x.shape[-1]
    x2 = x.reshape(-1, k)
    if scale.numel() == 1:
        return x2, ops.broadcast_f32(scale.reshape(1).to(torch.float32).contiguous(), x2.shape[0])
    else:
        if scale.shape[-1] != 1 and scale.dim() == x.dim():
            raise NotImplementedError("daxq leaf quantisers take one scale per row (or one per tensor)")
        s = scale.to(torch.float32).expand(*x.shape[:-1], 1).reshape(-1)
    return x2, s.contiguous()


def quantize_to_fp8(x: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    if dtype not in FP8_ALLOWED_DTYPES:
        raise NotImplementedError(f"daxq implements float8_e4m3fn and float8_e5m2, got {dtype}")
    x2, s = _rows_and_scale(x, scale)
    q = ops.quantize_rows_e4m3(x2, s) if dtype == torch.float8_e4m3fn else ops.quantize_rows_e5m2(x2, s)
    return q.view(dtype).view(x.shape)


def quantize_to_int8(x: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    if dtype != torch.int8:
        raise NotImplementedError(f"daxq implements int8 only, got {dtype}")
    x2, s = _rows_and_scale(x, scale)
    return ops.quantize_rows_i8(x2, s).view(x.shape)
