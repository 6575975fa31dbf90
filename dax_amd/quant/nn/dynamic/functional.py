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


_ROUND_KIND = {torch.bfloat16: 1, torch.float16: 2, torch.float32: 0}  # how daxq_tensor_scale rounds the quotient


def _dynamic_quantize_func(
    input: Optional[torch.Tensor],
    block_size: List[int],
    target_dtype: torch.dtype,
    quant_max: Optional[Union[int, float, bool]] = None,
    eps: Optional[float] = None,
    scale_dtype: Optional[torch.dtype] = None,
    scale_fp32: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantises `input` block by block; returns (values in the input's shape, scales in the view shape of the
    reduction with every reduced dim kept as 1).  dax/quant/nn/dynamic/functional.py:54-148.

    Arguments as in the reference: ``quant_max`` divides the block's abs-max (it must be given: the reference calls
    ``float(quant_max)``, :126); ``eps`` floors the scale (:127; the reference's own default reads an attribute that
    does not exist, :107, so every caller passes it -- here None means ``finfo(scale_dtype).eps``); ``scale_dtype`` is
    the type the scale is returned in (None: the input's own, :104-105) and, through type promotion, decides the type
    the leaf quantiser computes in.  Quotient and floor are computed in the input's element type before the cast
    (:124-129).  ``scale_fp32`` (not a reference argument): quotient and floor stay in fp32, which is what is left of
    that chain when the reference's forward runs under its ``torch.compile`` decorator (linear.py:143).

    Which kernels run: blocks that lie along the last dimension only (per-token, last-dimension groups) with an fp32
    scale are rows of a matrix and take the one-pass row quantiser; a whole-tensor block takes the row statistics +
    single reduction; every other block shape, and scales of a 16-bit type, take the general strided kernels.
    """
    assert input.dtype in [torch.float32, torch.float16, torch.bfloat16], f"Unsupported input dtype: {input.dtype}"
    if scale_dtype is None:
        scale_dtype = input.dtype
    if scale_dtype not in (torch.float32, torch.float16, torch.bfloat16):
        raise NotImplementedError(f"Unsupported scale dtype {scale_dtype}")
    if eps is None:
        eps = torch.finfo(scale_dtype).eps
    assert len(block_size) == input.dim(), f"Got input dim:{input.dim()}, block_size: {block_size}"
    if target_dtype not in ops.FMT_OF_DTYPE:
        raise NotImplementedError(f"Unsupported dtype {target_dtype}")
    fmt = ops.FMT_OF_DTYPE[target_dtype]
    qmax = float(quant_max)  # (TypeError for None, as in the reference)
    eps = float(eps)
    if not qmax > 0 or not eps >= 0:
        raise ValueError(f"quant_max must be positive and eps not negative, got {quant_max} and {eps}")
    round_x = not scale_fp32
    view_shape, reduce_dims = _get_reduction_params(tuple(block_size), tuple(input.shape))
    after = [1 if i in reduce_dims else v for i, v in enumerate(view_shape)]
    x = input if input.is_contiguous() else input.contiguous()  # the reference's .view needs that layout anyway
    as_dtype = (lambda q: q) if fmt == "i8" else (lambda q: q.view(target_dtype))
    if input.numel() == 0:
        return as_dtype(torch.empty(input.shape, dtype=torch.int8 if fmt == "i8" else torch.uint8, device=input.device)), \
            torch.empty(after, dtype=scale_dtype, device=input.device)
    fp32_scale = scale_dtype == torch.float32
    if tuple(block_size) == tuple(input.shape) and not _is_per_token(block_size, input.shape) and fp32_scale:
        q, s1 = _per_tensor_quantize(x, fmt, qmax, eps, round_x)
        return as_dtype(q).view(input.shape), s1.view(after)
    g = block_size[-1] if len(block_size) else 1
    if all(b == 1 for b in block_size[:-1]) and g > 1 and input.dim() >= 1 and fp32_scale:
        # rows of the [numel / g, g] view: per-token (g = K) and last-dimension groups
        x2 = x.view(-1, g)
        if qmax == ops.QMAX[fmt] and eps == ops.EPS_F32:
            q, s = getattr(ops, "act_quant_" + fmt)(x2, scale_fp32)
        else:
            q, s = ops.act_quant_rows(x2, fmt, qmax, eps, round_x)
        return as_dtype(q[:, :g]).reshape(input.shape), s.view(after)
    reduced = [1 if i in reduce_dims else 0 for i in range(len(view_shape))]
    s = ops.block_scale(x, view_shape, reduced, qmax, round_x, eps)
    if not fp32_scale:
        # the scale the quantiser sees is the one the caller gets: rounded to scale_dtype (:128-129), then widened
        s_out = s.to(scale_dtype)
        s = s_out.to(torch.float32)
    else:
        s_out = s
    q = ops.block_quantize(x, view_shape, reduced, s, fmt, scale_dtype)
    return as_dtype(q).view(input.shape), s_out.view(after)


def per_tensor_scale(x2: torch.Tensor, quant_max: float, eps: float = ops.EPS_F32, round_x: bool = True):
    """(scale fp32 [1], the same value once per row of x2) of the whole matrix x2; quotient and floor are rounded to
    x2's own element type, as the eager dtype chain does (:124-129), unless ``round_x`` is off."""
    lo, hi = ops.row_minmax(x2)
    return ops.tensor_scale(lo, hi, quant_max, _ROUND_KIND[x2.dtype] if round_x else 0, x2.shape[0], eps)


def _per_tensor_quantize(x, fmt, quant_max, eps=ops.EPS_F32, round_x=True):
    k = x.shape[-1] if x.dim() else 1
    x2 = x.reshape(-1, k)
    s1, rows = per_tensor_scale(x2, quant_max, eps, round_x)
    return getattr(ops, "quantize_rows_" + fmt)(x2, rows), s1


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
