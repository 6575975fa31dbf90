"""Dynamic (per call) activation quantisation.

Same entry points as dax/quant/nn/dynamic/functional.py:13-206.  The per-token scheme, the
one on the DiT hot path, is a single fused HIP kernel (row abs-max with wavefront shuffles,
bf16-rounded scale floored at 2^-23, quantise from registers).  The scale recipe follows the
reference's eager dtype chain for a bf16 input: the division by quant_max and the clamp
happen in bf16, and only then is the scale widened to fp32 (:124-129).  The per-tensor scheme
(one block = the whole tensor) runs the row statistics kernel, a single-workgroup reduction to
the scalar scale by the same rule, and the leaf quantiser with that scale.
"""
from typing import List, Optional, Tuple, Union

import torch

from .... import ops
from ...qscheme import FP8_QSCHEME, INT8_QSCHEME, get_block_size, per_tensor_symmetric
from ..quantized.functional import FP8_ALLOWED_DTYPES


def _get_reduction_params(block_size, input_size):
    """View shape and the dims to reduce so that every block of `block_size` collapses to
    one element (dax/quant/nn/dynamic/functional.py:13-51).

    A dim whose block spans it entirely is reduced in place; a dim split into several
    blocks becomes (n_blocks, block) with the second reduced; block 1 is left alone.
    """
    assert len(block_size) == len(input_size)
    view_shape, reduce_dims = [], []
    for blk, size in zip(block_size, input_size):
        if blk != size and blk > 1:
            assert size % blk == 0, (
                f"Expecting input size at {len(view_shape)} dimension: {size} to be divisible by block_size: {blk}")
            view_shape += [size // blk, blk]
            reduce_dims.append(len(view_shape) - 1)
        else:
            view_shape.append(size)
            if blk != 1:
                reduce_dims.append(len(view_shape) - 1)
    return view_shape, reduce_dims


def _is_per_token(block_size, shape) -> bool:
    return tuple(block_size) == (1,) * (len(shape) - 1) + (shape[-1],)


def _dynamic_quantize_func(
    input: Optional[torch.Tensor],
    block_size: List[int],
    target_dtype: torch.dtype,
    quant_max: Optional[Union[int, float, bool]] = None,
    eps: Optional[float] = None,
    scale_dtype: Optional[torch.dtype] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantises `input` block by block; returns (values in the input's shape, scales with
    every reduced dim kept as 1).  dax/quant/nn/dynamic/functional.py:54-148."""
    assert input.dtype in [torch.float32, torch.float16, torch.bfloat16], f"Unsupported input dtype: {input.dtype}"
    assert len(block_size) == input.dim(), f"Got input dim:{input.dim()}, block_size: {block_size}"
    if target_dtype not in FP8_ALLOWED_DTYPES and target_dtype != torch.int8:
        raise NotImplementedError(f"Unsupported dtype {target_dtype}")
    per_tensor = tuple(block_size) == tuple(input.shape)
    if not (per_tensor or _is_per_token(block_size, input.shape)):
        raise NotImplementedError("daxq implements the per-token and per-tensor dynamic schemes; grouped blocks are not built")
    if scale_dtype not in (None, torch.float32) or (eps is not None and eps != torch.finfo(torch.float32).eps):
        raise NotImplementedError("daxq kernels produce fp32 scales floored at float32 eps")
    if per_tensor and not _is_per_token(block_size, input.shape):
        return _per_tensor_quantize(input, target_dtype, float(quant_max))
    k = input.shape[-1]
    x2 = input.reshape(-1, k)
    if target_dtype == torch.int8:
        q, s = ops.act_quant_i8(x2)
    elif target_dtype == torch.float8_e5m2:
        q, s = ops.act_quant_e5m2(x2)
        q = q.view(torch.float8_e5m2)
    else:
        q, s = ops.act_quant_e4m3(x2)
        q = q.view(torch.float8_e4m3fn)
    return q[:, :k].view(input.shape), s.view(*input.shape[:-1], 1)


def per_tensor_scale(x2: torch.Tensor, quant_max: float):
    """(scale fp32 [1], the same value once per row of x2) of the whole bf16 matrix x2."""
    lo, hi = ops.row_minmax(x2)
    return ops.tensor_scale(lo, hi, quant_max, True, x2.shape[0])


def _per_tensor_quantize(input, target_dtype, quant_max):
    k = input.shape[-1]
    x2 = input.reshape(-1, k)
    if x2.stride(1) != 1:
        x2 = x2.contiguous()
    s1, rows = per_tensor_scale(x2, quant_max)
    if target_dtype == torch.int8:
        q = ops.quantize_rows_i8(x2, rows)
    elif target_dtype == torch.float8_e5m2:
        q = ops.quantize_rows_e5m2(x2, rows).view(torch.float8_e5m2)
    else:
        q = ops.quantize_rows_e4m3(x2, rows).view(torch.float8_e4m3fn)
    return q.view(input.shape), s1.view((1,) * input.dim())


def dynamic_quantize_to_fp8(
    input_float: torch.Tensor,
    qscheme: str = per_tensor_symmetric,
    block_size: List[int] = None,
    target_dtype: Optional[torch.dtype] = torch.float8_e4m3fn,
    scale_dtype: Optional[torch.dtype] = torch.float32,
):
    if block_size is None:
        assert qscheme is not None and qscheme in FP8_QSCHEME, f"Invalid qscheme: {qscheme}, expected {FP8_QSCHEME}"
        block_size = get_block_size(input_float.shape, qscheme)
    if target_dtype not in FP8_ALLOWED_DTYPES:
        raise NotImplementedError(f"Unsupported dtype {target_dtype} for dynamic_quantize_to_fp8")
    return _dynamic_quantize_func(
        input_float, block_size=block_size, target_dtype=target_dtype,
        quant_max=torch.finfo(target_dtype).max, eps=torch.finfo(scale_dtype).eps, scale_dtype=scale_dtype)


def dynamic_quantize_to_int8(
    input_float: torch.Tensor,
    qscheme: str = per_tensor_symmetric,
    block_size: List[int] = None,
    target_dtype: Optional[torch.dtype] = torch.int8,
    scale_dtype: Optional[torch.dtype] = torch.float32,
):
    if block_size is None:
        assert qscheme is not None and qscheme in INT8_QSCHEME, f"Invalid qscheme: {qscheme}, expected {INT8_QSCHEME}"
        block_size = get_block_size(input_float.shape, qscheme)
    if target_dtype != torch.int8:
        raise NotImplementedError(f"Unsupported dtype {target_dtype} for dynamic_quantize_to_int8")
    return _dynamic_quantize_func(
        input_float, block_size=block_size, target_dtype=target_dtype,
        quant_max=torch.iinfo(target_dtype).max, eps=torch.finfo(scale_dtype).eps, scale_dtype=scale_dtype)
