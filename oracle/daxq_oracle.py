"""CPU oracle for the DAX dynamic W8A8 linear (INT8 and FP8-e4m3fn).

TEST INFRASTRUCTURE ONLY.  This file is the checker that the HIP kernels are
compared against; nothing in the shipped package may import or call it.  It is
used by ``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline``
leg of ``bench.py``.

Every function restates, with plain PyTorch CPU ops and the same dtype chain as
the reference's *eager* execution, the reference lines cited in its docstring
(paths are relative to the reference checkout).  The reference package itself is
never imported: it raises at import time on a non-CUDA torch
(dax/quant/nn/quantized/linear.py:21-25).

How each function is pinned (see tests/test_oracle_*.py):

* act_scale                exhaustive over every finite bf16 amax against the
                           bit-level C closed form (oracle/daxq_oracle_c.c)
* quantize_to_int8         C closed form on every bf16 x for sampled reachable
                           scales + special rows (zero row, +-amax -> +-127)
* quantize_to_fp8          torch's f32->e4m3fn cast against the bit-level C
                           encoder on all 2^16 bf16 inputs x many scales and on
                           a dense sweep of f32 bit patterns; tie / saturation
                           / subnormal known answers
* weight_scale / quant     C closed form, brute force on small matrices
* int_mm                   numpy int64 brute force, adversarial +-127 / -128
* linear_int8 epilogue     C closed form bf16(bf16(f32(acc)*sx*sw)+bias)
* layernorm_affine_bf16    float64 statistics on random and constant rows; the bf16
  gelu_tanh_bf16           result may differ from an exact evaluation by one ulp
                           at rounding boundaries (floating point: tolerance
                           stated in the tests); gelu checked on every bf16 input
* act_scale_per_tensor /   reduce to the per-row functions above on the tensor flattened
  weight_scale_per_tensor  to one row (tests/test_oracle_pins.py)
* linear_fp8 /             float64 evaluation from the decoded bytes with one final rounding
  static_linear_fp8 /      (tests/test_oracle_pins.py: all four e4m3fn / e5m2 operand pairs, per-row and
  scaled_mm_fp32           per-column scales, a bias as large as the outputs): at most one bf16 step
                           apart on < 1 % of the outputs, which a dropped bias, a second rounding or
                           the other format's decoding all break; uniform scales reduce to the library
                           routine torch._scaled_mm on CPU, called on the oracle's own operands.  The
                           summation order of the reference's GPU matmul (cuBLASLt fast-accum) is not
                           fixed, so GPU comparisons against it use the 2e-2 relative-L2 tolerance
* dynamic_quantize         every block of every scheme equals the per-row rule on the block flattened
                           to one row (brute force over blocks); fp16 scales exhaustive over every
                           finite fp16 abs-max against numpy; fp32 / fp16 inputs against numpy fp32
                           arithmetic and the C fp8 encoders
* linear_int8_float_       float64 matmul on the bf16 de-quantised weight (tolerance: the float
  fallback                 matmul's summation order is the library's)
* act_scale_fp32           closed form max(f32(amax) / qmax, eps) in numpy float32 over every finite bf16 / fp16
                           abs-max; PARITY UNPINNED against the reference as it runs compiled on an NVIDIA GPU
                           (which instruction the generated code divides with cannot be observed here)
* dynamic_quantize with    quant_max / eps / scale_dtype other than the wrappers': numpy restatement of the
  caller's arguments       dtype chain element by element (scale in x's type, cast, promoted arithmetic)
"""

from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

INT8_QMAX = 127  # torch.iinfo(torch.int8).max      dynamic/functional.py:199
E4M3_QMAX = 448.0  # torch.finfo(torch.float8_e4m3fn).max   dynamic/functional.py:170
E5M2_QMAX = 57344.0  # torch.finfo(torch.float8_e5m2).max (the FP8 qconfig's default activation dtype)
EPS = torch.finfo(torch.float32).eps  # 2**-23     dynamic/functional.py:171,200


# --------------------------------------------------------------------------- #
# host-side shape helpers
# --------------------------------------------------------------------------- #
def get_block_size(shape: Tuple[int, ...], qscheme: str) -> Tuple[int, ...]:
    """dax/quant/qscheme.py:10-26."""
    kind = qscheme.rsplit(".", 1)[-1]
    if kind == "per_tensor_symmetric":
        return tuple(shape)
    if kind == "per_token_symmetric":
        return (1,) * (len(shape) - 1) + (shape[-1],)
    if kind == "per_channel_symmetric":
        return tuple(shape[:-1]) + (1,)
    raise ValueError(f"Unsupported QScheme: {qscheme}")


# --------------------------------------------------------------------------- #
# activation quantisation (per token)
# --------------------------------------------------------------------------- #
def act_scale(x: torch.Tensor, qmax: float) -> torch.Tensor:
    """Per-token scale, eager dtype chain.  dax/quant/nn/dynamic/functional.py:124-135.

    ``x`` is [M, K] in its original dtype (bf16 on the hot path).  The division
    and the clamp happen in x's dtype; only then is the scale widened to fp32.
    Returns fp32 [M, 1].
    """
    amax = x.abs().amax(dim=-1, keepdim=False)  # :124
    scale = amax / float(qmax)  # :126
    scale = torch.clamp(scale, min=EPS)  # :127
    if scale.dtype != torch.float32:  # :128-129
        scale = scale.to(torch.float32)
    return scale.view(-1, 1)  # :131-135


def quantize_to_int8(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """dax/quant/nn/quantized/functional.py:17-20 (reciprocal-multiply, RNE, clamp)."""
    return torch.clamp(torch.round(x * (1.0 / scale)), -128, 127).to(torch.int8)


def quantize_to_fp8(x: torch.Tensor, scale: torch.Tensor, dtype: torch.dtype = torch.float8_e4m3fn) -> torch.Tensor:
    """dax/quant/nn/quantized/functional.py:11-13 (true division, clamp to the dtype's max, RNE cast)."""
    qmax = torch.finfo(dtype).max
    return (x / scale).clamp(-qmax, qmax).to(dtype)


def act_quant_int8(x: torch.Tensor, scale_fp32: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """dynamic_quantize_to_int8, per-token.  dynamic/functional.py:181-206, :54-148.  scale_fp32: act_scale_fp32."""
    x2 = x.reshape(-1, x.shape[-1])
    s = act_scale_fp32(x2, INT8_QMAX) if scale_fp32 else act_scale(x2, INT8_QMAX)
    return quantize_to_int8(x2, s), s


def act_quant_e4m3(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """dynamic_quantize_to_fp8, per-token, e4m3fn.  dynamic/functional.py:152-177."""
    x2 = x.reshape(-1, x.shape[-1])
    s = act_scale(x2, E4M3_QMAX)
    return quantize_to_fp8(x2, s), s


def act_quant_e5m2(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """dynamic_quantize_to_fp8, per-token, e5m2 (qconfig.py:85-87 default).  dynamic/functional.py:152-177."""
    x2 = x.reshape(-1, x.shape[-1])
    s = act_scale(x2, E5M2_QMAX)
    return quantize_to_fp8(x2, s, torch.float8_e5m2), s


def get_reduction_params(block_size, input_size):
    """View shape and reduced dims of a block scheme.  dax/quant/nn/dynamic/functional.py:13-51: a dim that is
    split into several blocks becomes (n_blocks, block) with the second reduced; a dim the block spans is
    reduced in place; block 1 keeps the dim."""
    assert len(block_size) == len(input_size)
    view, dims = [], []
    for blk, size in zip(block_size, input_size):
        if blk != size and blk > 1:
            assert size % blk == 0
            view += [size // blk, blk]
            dims.append(len(view) - 1)
        else:
            view.append(size)
            if blk != 1:
                dims.append(len(view) - 1)
    return view, dims


def dynamic_quantize(x: torch.Tensor, block_size, target_dtype: torch.dtype, quant_max=None, eps=None,
                     scale_dtype: Optional[torch.dtype] = torch.float32,
                     fused_chain: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """``_dynamic_quantize_func`` for any block shape, any of the input dtypes it accepts (fp32 / fp16 / bf16) and
    any quant_max / eps / scale_dtype.  dax/quant/nn/dynamic/functional.py:54-148.  The defaults are what its two
    wrappers pass (:152-206): quant_max of the target dtype, eps = eps of the scale dtype, fp32 scales.
    Returns (values in x's shape, scales with every reduced dim kept as 1, in the view shape of get_reduction_params).

    fused_chain: ``act_scale_fp32`` below applied per block -- abs-max widened to fp32 first, quotient and floor in fp32."""
    if quant_max is None:
        quant_max = INT8_QMAX if target_dtype == torch.int8 else torch.finfo(target_dtype).max
    if scale_dtype is None:  # :104-105
        scale_dtype = x.dtype
    if eps is None:
        eps = torch.finfo(scale_dtype).eps
    view, dims = get_reduction_params(tuple(block_size), tuple(x.shape))
    xv = x.view(view)  # :121
    amax = xv.abs().amax(dim=dims, keepdim=False) if dims else xv.abs()  # :124
    if fused_chain:
        amax = amax.to(torch.float32)
    scale = torch.clamp(amax / float(quant_max), min=eps)  # :126-127, in x's dtype
    if scale.dtype != scale_dtype:  # :128-129
        scale = scale.to(scale_dtype)
    after = list(view)
    for i in dims:  # :131-135
        after[i] = 1
    scale = scale.view(after)
    if target_dtype == torch.int8:  # :137-148
        return quantize_to_int8(xv, scale).view(x.shape), scale
    return quantize_to_fp8(xv, scale, target_dtype).view(x.shape), scale


def act_scale_fp32(x: torch.Tensor, qmax: float, eps: float = EPS) -> torch.Tensor:
    """The per-token scale with quotient and floor in fp32: ``max(f32(rowamax) / qmax, eps)``, fp32 [M, 1].

    The reference's forward carries ``@torch.compile`` (dax/quant/nn/dynamic/linear.py:143).  A code generator that
    fuses dynamic/functional.py:124-129 computes in fp32 and does not materialise the bf16 quotient (torch's inductor
    leaves such casts out unless told to emulate them), so on an NVIDIA run the scale is this fp32 value.  The
    division here is IEEE; what instruction the generated code divides with is not something this build can observe.
    """
    amax = x.abs().amax(dim=-1, keepdim=False).to(torch.float32)
    return torch.clamp(amax / float(qmax), min=eps).view(-1, 1)


# --------------------------------------------------------------------------- #
# weight quantisation (per output channel, one time)
# --------------------------------------------------------------------------- #
def weight_scale(w: torch.Tensor, qmax: float) -> torch.Tensor:
    """PerChannelMinMaxObserver + _calculate_qparams.

    dax/quant/quantization/observer.py:284-312 (fp32 row min/max) and :97-134
    (amax / qmax, floor at eps) -- all in fp32, no bf16 rounding.  Returns fp32 [N].
    """
    y = w.detach().to(torch.float32).flatten(1)  # :298-299
    lo, hi = torch.aminmax(y, dim=1)  # :301
    amax = torch.max(-lo, hi)  # :123
    scale = amax / float(qmax)  # :125
    return torch.max(scale, torch.tensor([EPS], dtype=torch.float32))  # :126


def weight_quant_int8(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """dax/quant/nn/dynamic/linear.py:276-299 with the int8 leaf quantiser."""
    s = weight_scale(w, INT8_QMAX)
    return quantize_to_int8(w, s.view(-1, 1)), s.view(1, -1)


def weight_quant_fp8(w: torch.Tensor, dtype: torch.dtype = torch.float8_e4m3fn) -> Tuple[torch.Tensor, torch.Tensor]:
    """dax/quant/nn/dynamic/linear.py:276-299 with the fp8 leaf quantiser (either of FP8_ALLOWED_DTYPES)."""
    s = weight_scale(w, torch.finfo(dtype).max)
    return quantize_to_fp8(w, s.view(-1, 1), dtype), s.view(1, -1)


def weight_quant_e4m3(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    return weight_quant_fp8(w, torch.float8_e4m3fn)


def dequant_weight(qweight: torch.Tensor, wscale: torch.Tensor, out_dtype=torch.bfloat16) -> torch.Tensor:
    """Linear.weight property.  dax/quant/nn/dynamic/linear.py:139-141."""
    return qweight.to(out_dtype) * wscale.T.to(out_dtype)


# --------------------------------------------------------------------------- #
# GEMM + epilogue
# --------------------------------------------------------------------------- #
def int_mm(xq: torch.Tensor, wq: torch.Tensor) -> torch.Tensor:
    """int8 [M,K] x int8 [N,K]^T -> int32 [M,N], exact.

    dax/quant/nn/dynamic/linear.py:218-220 (out_dtype(aten.mm, int32, ...)).
    torch._int_mm is the library routine of the CPU path; it is
    exact integer arithmetic, so any summation order gives the same bits.
    """
    return torch._int_mm(xq.contiguous(), wq.t())


def epilogue_int8(acc: torch.Tensor, sx: torch.Tensor, sw: torch.Tensor,
                  bias: Optional[torch.Tensor], out_dtype=torch.bfloat16) -> torch.Tensor:
    """dax/quant/nn/dynamic/linear.py:214,221-228.

    int32 * fp32 -> fp32 (acc converted RNE), * weight_scale fp32, cast to
    out_dtype, then a second rounding when the bf16 bias is added.
    """
    m, n = acc.shape
    out = acc * sx.reshape(-1, 1).expand(m, n)  # :214,:221
    out = out * sw.reshape(1, -1)  # :222
    if out.dtype != out_dtype:  # :225-226
        out = out.to(out_dtype)
    if bias is not None:  # :227-228
        out = out + bias
    return out


def linear_int8(x: torch.Tensor, qweight: torch.Tensor, wscale: torch.Tensor,
                bias: Optional[torch.Tensor], row_chunk: int = 8192,
                keep_acc: bool = True, scale_fp32: bool = False) -> Dict[str, torch.Tensor]:
    """Whole INT8 forward.  dax/quant/nn/dynamic/linear.py:180-228.

    Processes rows in chunks so that the int32 accumulator of the big shapes is
    never resident in full unless ``keep_acc``.  Returns xq, sx, (acc), out.
    """
    prev = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    xq, sx = act_quant_int8(x2, scale_fp32)
    outs, accs = [], []
    for r0 in range(0, x2.shape[0], row_chunk):
        acc = int_mm(xq[r0:r0 + row_chunk], qweight)
        outs.append(epilogue_int8(acc, sx[r0:r0 + row_chunk], wscale, bias, x.dtype))
        if keep_acc:
            accs.append(acc)
    out = torch.cat(outs, 0).view(*prev, qweight.shape[0])
    res = {"xq": xq, "sx": sx, "out": out}
    if keep_acc:
        res["acc"] = torch.cat(accs, 0)
    return res


def scaled_mm_fp32(xq: torch.Tensor, qweight: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
                   bias: Optional[torch.Tensor], out_dtype: torch.dtype, row_chunk: int = 8192) -> torch.Tensor:
    """``torch._scaled_mm(xq, qweight.T, scale_a, scale_b, bias, out_dtype)`` restated in fp32.

    dax/quant/nn/dynamic/linear.py:155-173 and dax/quant/nn/quantized/linear.py:105-113 call it with
    row-wise scales ([M,1] x [1,N], CUDA only) or per-tensor scales (one element each, the case the CPU
    routine implements).  Semantics: out_dtype( (sum_k a*b in fp32) * scale_a * scale_b + bias ), one
    rounding.  The summation order of the reference (cuBLASLt, use_fast_accum=True) is not specified.
    """
    wf = qweight.to(torch.float32)
    sa = scale_a.to(torch.float32).reshape(-1, 1)
    sb = scale_b.to(torch.float32).reshape(1, -1)
    outs = []
    for r0 in range(0, xq.shape[0], row_chunk):
        acc = xq[r0:r0 + row_chunk].to(torch.float32) @ wf.t()
        o = acc * (sa[r0:r0 + row_chunk] if sa.shape[0] > 1 else sa) * sb
        if bias is not None:
            o = o + bias.to(torch.float32)
        outs.append(o.to(out_dtype))
    return torch.cat(outs, 0)


def linear_fp8(x: torch.Tensor, qweight: torch.Tensor, wscale: torch.Tensor, bias: Optional[torch.Tensor],
               act_dtype: torch.dtype = torch.float8_e4m3fn, per_tensor: bool = False,
               out_dtype: Optional[torch.dtype] = None, row_chunk: int = 8192,
               scale_fp32: bool = False) -> Dict[str, torch.Tensor]:
    """Whole FP8 forward of the dynamic module.  dax/quant/nn/dynamic/linear.py:145-178.

    ``qweight`` is float8_e4m3fn or float8_e5m2 [N,K]; ``act_dtype`` the activation format (the FP8 qconfig's
    default is float8_e5m2, qconfig.py:85-87).  per-token + per-channel: scale_a [M,1], scale_b [1,N], the matmul
    writes bf16 with a bf16 bias (:111-116, :166-170) and the result is cast to the module's out_dtype afterwards
    (:177-178).  per-tensor + per-tensor: one-element scales and the matmul writes out_dtype directly.
    ``out_dtype`` defaults to x's dtype (the module takes it from the float weight, :263).
    """
    out_dtype = out_dtype or x.dtype
    prev = x.shape[:-1]
    x2 = x.reshape(-1, x.shape[-1])
    qmax = torch.finfo(act_dtype).max
    if per_tensor:
        sx = act_scale_per_tensor(x2, qmax)
        mm_dtype = out_dtype
    else:
        sx = act_scale_fp32(x2, qmax) if scale_fp32 else act_scale(x2, qmax)
        mm_dtype = torch.bfloat16
    xq = quantize_to_fp8(x2, sx, act_dtype)
    out = scaled_mm_fp32(xq, qweight, sx, wscale, None if bias is None else bias.to(mm_dtype), mm_dtype, row_chunk)
    if out.dtype != out_dtype:
        out = out.to(out_dtype)
    return {"xq": xq, "sx": sx, "out": out.view(*prev, qweight.shape[0])}


def linear_e4m3(x: torch.Tensor, qweight: torch.Tensor, wscale: torch.Tensor,
                bias: Optional[torch.Tensor], row_chunk: int = 8192,
                act_dtype: torch.dtype = torch.float8_e4m3fn) -> Dict[str, torch.Tensor]:
    """The per-token / per-channel FP8 forward of a bf16 module (the benchmark's FP8 configuration)."""
    return linear_fp8(x, qweight, wscale, bias, act_dtype=act_dtype, row_chunk=row_chunk)


def takes_float_fallback(m: int, k: int, n: int) -> bool:
    """The shapes the reference's INT8 forward hands to a float matmul when it runs un-compiled:
    M <= 16, or K or N not a positive multiple of 8.  dax/quant/nn/dynamic/linear.py:186-194."""
    return not (m > 16 and k % 8 == 0 and k > 0 and n % 8 == 0 and n > 0)


def linear_int8_float_fallback(x: torch.Tensor, qweight: torch.Tensor, wscale: torch.Tensor,
                               bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``F.linear(input, self.weight, self.bias)`` on the de-quantised weight.  dax/quant/nn/dynamic/linear.py:195-202,
    taken only outside a compiled graph (``not is_compiling()``).  The matmul is a float one in the module's dtype;
    its summation order is the library's, so comparisons use a tolerance."""
    w = dequant_weight(qweight, wscale, x.dtype)
    return torch.nn.functional.linear(x, w, None if bias is None else bias.to(x.dtype))


# --------------------------------------------------------------------------- #
# synthetic workload of the benchmark configs (shared by tests and bench.py)
# --------------------------------------------------------------------------- #
def make_inputs(m: int, k: int, n: int, seed: int = 0):
    """Seeded synthetic X, W, bias with 1 % outlier channels (x20), all bf16, on CPU."""
    g = torch.Generator("cpu").manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    idx = torch.randperm(k, generator=g)[: max(1, round(0.01 * k))]
    x[:, idx] *= 20
    x = x.bfloat16()
    w = (torch.randn(n, k, generator=g) * 0.02).bfloat16()
    b = (torch.randn(n, generator=g) * 0.01).bfloat16()
    return x, w, b


# --------------------------------------------------------------------------- #
# producers in front of a quantised linear (what the fused kernels restate)
# --------------------------------------------------------------------------- #
def layernorm_affine_bf16(x: torch.Tensor, mul: Optional[torch.Tensor], add: Optional[torch.Tensor],
                          rows_per_group: int, eps: float) -> torch.Tensor:
    """``(norm(x.float()) * mul + add).type_as(x)`` with an fp32 LayerNorm without affine parameters and
    one (mul, add) pair of fp32 [K] vectors per group of ``rows_per_group`` consecutive rows.

    Operation order of dax/adapters/wan/transformer_adapter.py:151-153 (mul = 1 + scale, add = shift);
    with mul = weight, add = bias and one group it is an affine fp32 LayerNorm cast back to bf16.

    torch's CPU kernel evaluates ``x * rstd - mean * rstd``; for a row whose offset is fifty or more times its spread
    that difference cancels and outputs next to zero lose digits, where ``(x - mean) * rstd`` (torch's GPU kernel)
    does not: tests of such rows compare with a float64 evaluation instead (tests/test_gpu_fused.py).
    """
    m, k = x.shape
    y = torch.nn.functional.layer_norm(x.float(), (k,), None, None, eps)
    g = torch.arange(m) // rows_per_group
    if mul is not None:
        y = y * mul.float().reshape(-1, k)[g]
    if add is not None:
        y = y + add.float().reshape(-1, k)[g]
    return y.to(x.dtype)


def gelu_tanh_bf16(x: torch.Tensor) -> torch.Tensor:
    """``gelu(x, approximate="tanh")`` of a bf16 tensor: evaluated in fp32, rounded once to bf16
    (the activation between the two FFN linears of the DiT)."""
    return torch.nn.functional.gelu(x.float(), approximate="tanh").to(x.dtype)


# --------------------------------------------------------------------------- #
# per-tensor schemes and the static FP8 linear
# --------------------------------------------------------------------------- #
def act_scale_per_tensor(x: torch.Tensor, qmax: float) -> torch.Tensor:
    """Dynamic per-tensor scale, eager dtype chain: the block of dax/quant/qscheme.py:10-26 is the whole
    tensor, so dax/quant/nn/dynamic/functional.py:124-129 reduces over every dimension.  fp32 [1]."""
    amax = x.abs().amax()
    scale = torch.clamp(amax / float(qmax), min=EPS)
    return scale.to(torch.float32).reshape(1)


def weight_scale_per_tensor(w: torch.Tensor, qmax: float) -> torch.Tensor:
    """MinMaxObserver + _calculate_qparams: dax/quant/quantization/observer.py:200-214 and :97-134, fp32 [1]."""
    lo, hi = torch.aminmax(w.detach().to(torch.float32))
    amax = torch.max(-lo, hi)
    return torch.max(amax / float(qmax), torch.tensor([EPS], dtype=torch.float32)).reshape(1)


def linear_int8_schemes(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], act_per_tensor: bool,
                        weight_per_tensor: bool) -> Dict[str, torch.Tensor]:
    """INT8 forward for any of the four scheme pairs of dax/quant/nn/dynamic/linear.py:180-228 (the scalar
    scales broadcast in :214 and :222)."""
    x2 = x.reshape(-1, x.shape[-1])
    sw = weight_scale_per_tensor(w, INT8_QMAX) if weight_per_tensor else weight_scale(w, INT8_QMAX)
    qw = quantize_to_int8(w, sw.reshape(-1, 1))
    if act_per_tensor:
        sx = act_scale_per_tensor(x2, INT8_QMAX)
        xq = quantize_to_int8(x2, sx)
        sx_rows = sx.expand(x2.shape[0])
    else:
        xq, sx = act_quant_int8(x2)
        sx_rows = sx.reshape(-1)
    acc = int_mm(xq, qw)
    out = epilogue_int8(acc, sx_rows, sw.expand(w.shape[0]) if sw.numel() == 1 else sw, bias, x.dtype)
    return {"xq": xq, "sx": sx, "qw": qw, "sw": sw, "acc": acc, "out": out.view(*x.shape[:-1], w.shape[0])}


def static_linear_fp8(x: torch.Tensor, input_scale: torch.Tensor, qweight: torch.Tensor, wscale: torch.Tensor,
                      bias: Optional[torch.Tensor], act_dtype: torch.dtype = torch.float8_e4m3fn,
                      out_dtype: Optional[torch.dtype] = None) -> Dict[str, torch.Tensor]:
    """Static FP8 forward, dax/quant/nn/quantized/linear.py:91-118: leaf quantiser with the stored input scale
    (one element), then ``_scaled_mm`` restated in fp32 (accumulation order of the reference unspecified: tolerance).
    With a per-channel weight scale the input scale is expanded to [M,1] and the matmul writes bf16 (:98-104)."""
    out_dtype = out_dtype or x.dtype
    x2 = x.reshape(-1, x.shape[-1])
    xq = quantize_to_fp8(x2, input_scale.reshape(1), act_dtype)
    mm_dtype = torch.bfloat16 if wscale.numel() > 1 else out_dtype
    out = scaled_mm_fp32(xq, qweight, input_scale.reshape(1), wscale, None if bias is None else bias.to(mm_dtype), mm_dtype)
    if out.dtype != out_dtype:
        out = out.to(out_dtype)
    return {"xq": xq, "out": out.view(*x.shape[:-1], qweight.shape[0])}
