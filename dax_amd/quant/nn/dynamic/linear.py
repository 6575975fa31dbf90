"""Dynamic W8A8 ``Linear``: the module that takes the place of ``nn.Linear`` inside the DiT.

Drop-in for dax/quant/nn/dynamic/linear.py:27-341: same constructor signature, the same
persistent state (``qweight`` [N,K] int8 / float8_e4m3fn, ``weight_scale`` fp32 [1,N],
``bias``), the same ``from_float`` / ``get_qlinear`` / ``weight`` / ``extra_repr`` surface
and the same exceptions for invalid dtype / qscheme combinations.

What differs is where the arithmetic runs: ``forward`` is two HIP launches -- the fused
per-token quantiser and the MFMA GEMM with the scale / bias / bf16 epilogue -- and the
conversion in ``get_qlinear`` uses the HIP observer and leaf-quantiser kernels.  Numerics are
those of the reference's eager op sequence (:180-228 for INT8, :145-178 for FP8).

Control flow for small INT8 problems: the reference hands M <= 16, or K / N that are not
multiples of 8, to a float matmul on the de-quantised weight, but only when the forward is NOT
being compiled (:186-202, ``not is_compiling()``) -- and its forward carries a ``torch.compile``
decorator (:143), so as shipped every shape is quantised.  That is the default here too.
``Linear.uncompiled_small_shape_fallback = True`` (class or instance attribute) gives the
un-compiled behaviour instead: those shapes then run ``F.linear(input, self.weight, self.bias)``,
a plain library matmul on the cold path.
"""
from __future__ import annotations

import logging

import torch
from torch import Tensor, nn

from .... import ops
from ...qscheme import per_channel_symmetric, per_tensor_symmetric, per_token_symmetric
from .._derived import DerivedOperands
from .functional import FP8_ALLOWED_DTYPES

logger = logging.getLogger(__name__)


class QuantizedActivation:
    """An activation that has already been through the per-token quantiser.

    Produced by ``Linear.quantize_activation`` or by a fused producer kernel (LayerNorm multiply-add,
    GELU-tanh) and accepted by ``Linear.forward`` in place of the bf16 tensor, so that several linears
    reading the same activation (q / k / v) share one quantisation and a producer can hand its result
    over without the bf16 round trip through memory.  It is not a tensor: code between the producer
    and the linears may only pass it along.
    """

    __slots__ = ("xq", "sx", "prev_dims", "in_features", "dtype", "device")

    def __init__(self, xq: Tensor, sx: Tensor, prev_dims, in_features: int, dtype: torch.dtype):
        self.xq, self.sx, self.prev_dims, self.in_features, self.dtype = xq, sx, tuple(prev_dims), in_features, dtype
        self.device = xq.device

    @property
    def shape(self):
        return torch.Size(self.prev_dims + (self.in_features,))


_ACT_QUANT = {torch.int8: "act_quant_i8", torch.float8_e4m3fn: "act_quant_e4m3", torch.float8_e5m2: "act_quant_e5m2"}
_DYNAMIC_LINEAR = {torch.int8: "dynamic_linear_i8", torch.float8_e4m3fn: "dynamic_linear_e4m3",
                   torch.float8_e5m2: "dynamic_linear_e5m2_e4m3"}


class Linear(DerivedOperands, nn.Module):
    _FLOAT_MODULE = nn.Linear
    # False: every shape is quantised, as under the reference's own torch.compile decorator (:143); True: the
    # un-compiled reference's float matmul for M <= 16 or K / N not multiples of 8 (:186-202)
    uncompiled_small_shape_fallback = False
    # False: the activation scale is computed in the input's own element type and only then widened to fp32, the
    # reference's eager op sequence (dynamic/functional.py:124-129).  True: quotient and floor stay in fp32 -- what is
    # left of that sequence when the forward runs under the torch.compile decorator it carries (:143; the code generator
    # does not materialise the bf16 intermediate), which moves the scale of almost every token by up to half a bf16 step
    # and about 0.4 % of the int8 values by one.  Class or instance attribute; the fused producer kernels and the block
    # fusion built on them implement the eager form only.
    act_scale_fp32 = False

    def __init__(
        self,
        in_features: int,
        out_features: int,
        bias: bool = True,
        device=None,
        weight_dtype=None,
        input_dtype=None,
        out_dtype=None,
        weight_qscheme=None,
        input_qscheme=None,
    ) -> None:
        # --- which arithmetic: same acceptance rules as the reference constructor (:42-89)
        if weight_dtype in FP8_ALLOWED_DTYPES and input_dtype in FP8_ALLOWED_DTYPES:
            token_channel = input_qscheme == per_token_symmetric and weight_qscheme == per_channel_symmetric
            tensor_tensor = input_qscheme == per_tensor_symmetric and weight_qscheme == per_tensor_symmetric
            if not (token_channel or tensor_tensor):
                raise ValueError(
                    f"Invalid qscheme combination! input_qscheme: {input_qscheme}, weight_qscheme: {weight_qscheme}")
            compute_dtype = "FP8"
        elif weight_dtype == torch.int8 and input_dtype == torch.int8:
            compute_dtype = "INT8"
        else:
            raise ValueError(f"Unsupported dtype combination! weight_dtype: {weight_dtype}, input_dtype: {input_dtype}")

        # --- what the gfx950 kernels cover; anything else is reported as not implemented so
        #     that get_qlinear keeps the float module, as the reference does on NotImplementedError
        if input_qscheme not in (per_token_symmetric, per_tensor_symmetric) or \
                weight_qscheme not in (per_channel_symmetric, per_tensor_symmetric):
            raise NotImplementedError(
                "daxq implements per-token / per-tensor activations with per-channel / per-tensor weights; "
                f"got input_qscheme={input_qscheme}, weight_qscheme={weight_qscheme}")
        if out_dtype not in (None, torch.bfloat16, torch.float16, torch.float32):
            raise NotImplementedError(f"daxq kernels produce bfloat16, float16 or float32 outputs, got out_dtype={out_dtype}")
        out_dtype = out_dtype if out_dtype is not None else torch.bfloat16

        super().__init__()
        self.in_features = in_features
        self.out_features = out_features

        self.register_buffer(
            "qweight", torch.empty((out_features, in_features), device=device, dtype=weight_dtype), persistent=True)
        if bias:
            # the row-wise FP8 matmul writes bf16 and takes a bf16 bias whatever the module's dtype (:106-118)
            row_wise_fp8 = compute_dtype == "FP8" and weight_qscheme == per_channel_symmetric
            self.bias = nn.Parameter(torch.empty(out_features, device=device,
                                                 dtype=torch.bfloat16 if row_wise_fp8 else out_dtype))
        else:
            self.register_parameter("bias", None)
        # [1, N] per channel, [1] per tensor (:122-130)
        self.register_buffer(
            "weight_scale",
            torch.ones((1, out_features) if weight_qscheme == per_channel_symmetric else 1, device=device,
                       dtype=torch.float32),
            persistent=True)

        self.out_dtype = out_dtype
        self.weight_dtype = weight_dtype
        self.input_dtype = input_dtype
        self.compute_dtype = compute_dtype
        self.weight_qscheme = weight_qscheme
        self.input_qscheme = input_qscheme
        self._init_derived()

    # ------------------------------------------------------------------ derived views
    @property
    def weight(self):
        """De-quantised weight in out_dtype, [N,K] (:139-141)."""
        return self.qweight.to(self.out_dtype) * self.weight_scale.T.to(self.out_dtype)

    # ------------------------------------------------------------------ forward
    def quantize_activation(self, input: Tensor) -> QuantizedActivation:
        """Dynamic quantisation of ``input`` [..., K] in this module's activation dtype and scheme
        (:204-208, :146-150): one scale per token, or one for the whole tensor written out per token."""
        flat = input.view(-1, self.in_features)
        if flat.stride(-1) != 1:  # a view with strided columns: the reference's torch ops take it, the kernels want rows
            flat = flat.contiguous()
        if self.input_qscheme == per_token_symmetric:
            xq, sx = getattr(ops, _ACT_QUANT[self.input_dtype])(flat, self.act_scale_fp32)
        else:
            from .functional import per_tensor_scale

            _, sx = per_tensor_scale(flat, ops.QMAX[ops.FMT_OF_DTYPE[self.input_dtype]], round_x=not self.act_scale_fp32)
            xq = getattr(ops, "quantize_rows_" + ops.FMT_OF_DTYPE[self.input_dtype])(flat, sx, True)
        return QuantizedActivation(xq, sx, input.shape[:-1], self.in_features, self.input_dtype)

    def _takes_float_fallback(self, input) -> bool:
        if not self.uncompiled_small_shape_fallback or self.compute_dtype != "INT8" or torch.compiler.is_compiling():
            return False
        if isinstance(input, QuantizedActivation):
            return False
        m = input.numel() // max(self.in_features, 1)
        k, n = self.in_features, self.out_features
        return not (m > 16 and k % 8 == 0 and k > 0 and n % 8 == 0 and n > 0)

    # ------------------------------------------------------------------ the common case, prepared ahead
    # A bf16 per-token module whose stored state already is what the GEMM reads keeps (op name, weight bytes, weight scale
    # vector, bias, device) ready: every torch call in a forward costs the host a microsecond or two, and a small
    # linear's time is the host's.  The tensors alias the module's state, so in-place updates show through; the tuple
    # also remembers which state tensors it was built from and where they lived, and a forward that finds other ones
    # (a buffer or parameter replaced by assignment, by a hook of an off-loading framework, or through `.data`)
    # rebuilds it.  Whatever sets the state afresh (conversion, load_state_dict, .to()) rebuilds it too.
    _fast = None

    def refresh_derived(self) -> None:
        super().refresh_derived()
        self._build_fast()

    def _build_fast(self):
        object.__setattr__(self, "_fast", None)
        qw, ws, bp = self._buffers["qweight"], self._buffers["weight_scale"], self._parameters["bias"]
        if (qw.device.type != "cuda" or self.input_qscheme != per_token_symmetric or self.out_dtype != torch.bfloat16
                or self.weight_dtype == torch.float8_e5m2 or ws.numel() == 1 or ops.pad_k(qw.shape[1]) != qw.shape[1]
                or not qw.is_contiguous() or ops.is_tracing(qw) or torch.cuda.is_current_stream_capturing()):
            return None
        bias = None if bp is None else bp.detach()
        if bias is not None and (bias.dtype != torch.bfloat16 or not bias.is_contiguous() or bias.device != qw.device):
            return None
        # (plain data only: a module must stay deep-copyable, and a copy finds the addresses changed and rebuilds)
        fast = (_DYNAMIC_LINEAR[self.input_dtype], self._gemm_weight(), self._weight_scale_vector(), bias,
                qw.device, qw, ws, bp, qw.data_ptr(), ws.data_ptr(), 0 if bp is None else bp.data_ptr())
        object.__setattr__(self, "_fast", fast)
        return fast

    def _fast_is_current(self, f) -> bool:
        qw, ws, bp = self._buffers["qweight"], self._buffers["weight_scale"], self._parameters["bias"]
        return (qw is f[5] and ws is f[6] and bp is f[7] and qw.data_ptr() == f[8] and ws.data_ptr() == f[9]
                and (bp is None or bp.data_ptr() == f[10]))

    def forward(self, input) -> Tensor:
        fast = self._fast
        if (fast is not None and input.__class__ is Tensor and input.dtype is torch.bfloat16
                and not self.uncompiled_small_shape_fallback and not torch.compiler.is_compiling()):
            if not self._fast_is_current(fast):
                self.refresh_derived()
                fast = self._fast
        else:
            fast = None
        if fast is not None:
            op, wq, sw, bias, dev = fast[:5]
            op = getattr(ops, op)
            if input.device != dev:
                self._check_device(input.device)
            if input.dim() == 2 and input.stride(1) == 1:
                return op(input, wq, sw, bias, self.act_scale_fp32)
            flat = input.view(-1, self.in_features)
            if flat.stride(-1) != 1:
                flat = flat.contiguous()
            return op(flat, wq, sw, bias, self.act_scale_fp32).view(*input.shape[:-1], self.out_features)
        self._check_device(input.device)
        if self._takes_float_fallback(input):
            logger.warning("int8 matmul not taken for this combination of dimensions, float implementation instead. "
                           "M: %d, K: %d, N: %d", input.numel() // self.in_features, self.in_features, self.out_features)
            return torch.nn.functional.linear(input, self.weight, self.bias)
        # the kernels are inference-only (no autograd formula): the bias enters as a plain tensor
        bias = None if self.bias is None else self.bias.detach()
        if (not isinstance(input, QuantizedActivation) and self.input_qscheme == per_token_symmetric
                and input.dtype == torch.bfloat16 and self.out_dtype == torch.bfloat16
                and self.weight_dtype != torch.float8_e5m2):
            # the common case (a bf16 DiT): quantiser and GEMM behind one op call
            flat = input.view(-1, self.in_features)
            if flat.stride(-1) != 1:
                flat = flat.contiguous()
            out = getattr(ops, _DYNAMIC_LINEAR[self.input_dtype])(flat, self._gemm_weight(), self._weight_scale_vector(), bias,
                                                                  self.act_scale_fp32)
            return out.view(*input.shape[:-1], self.out_features)
        qa = input if isinstance(input, QuantizedActivation) else self.quantize_activation(input)
        if qa.dtype != self.input_dtype or qa.in_features != self.in_features:
            raise ValueError(f"quantised activation ({qa.dtype}, K={qa.in_features}) does not fit this linear "
                             f"({self.input_dtype}, K={self.in_features})")
        # What the matmul writes: INT8 scales in fp32 and casts to the module's dtype (:221-228); the row-wise FP8
        # matmul writes bf16 and the result is cast afterwards (:166-178); per-tensor FP8 writes the module's dtype.
        row_wise_fp8 = self.compute_dtype == "FP8" and self.input_qscheme == per_token_symmetric
        mm_dtype = torch.bfloat16 if row_wise_fp8 else self.out_dtype
        out = ops.linear_w8a8(qa.xq, qa.sx, self._gemm_weight(), self._weight_scale_vector(), bias,
                              ops.FMT_OF_DTYPE[self.input_dtype], ops.FMT_OF_DTYPE[self.weight_dtype], mm_dtype)
        out = out.view(*qa.prev_dims, self.out_features)
        if out.dtype != self.out_dtype:
            out = out.to(self.out_dtype)
        return out

    def extra_repr(self) -> str:
        s = f"in_features={self.in_features}, out_features={self.out_features}"
        if self.bias is None:
            s += ", bias=False"
        s += f", weight_scale={self.weight_scale}"
        return s

    # ------------------------------------------------------------------ conversion
    @classmethod
    @torch.no_grad()
    def get_qlinear(cls, mod, activation_post_process, weight_post_process, reserve_float_weight):
        """Builds the quantised module from a float ``nn.Linear`` (:240-309).

        The weight statistics, the per-channel scale and the quantised weight are computed by
        HIP kernels; a module that still lives on the CPU is staged through the current
        ROCm device and the results are moved back to where the module was.
        """
        if activation_post_process is None or activation_post_process.dtype == torch.float:
            raise ValueError("Input must be quantized!")
        try:
            qlinear = cls(
                mod.in_features,
                mod.out_features,
                mod.bias is not None,
                mod.weight.device,
                weight_post_process.dtype,
                activation_post_process.dtype,
                mod.weight.dtype,
                weight_post_process.qscheme,
                activation_post_process.qscheme,
            )
        except NotImplementedError as e:
            logger.warning("Quantized linear is not supported for this combination of arguments. "
                           "Falling back to float module. Message: %s", e)
            return mod

        home = mod.weight.device
        w = mod.weight.detach()
        if home.type != "cuda":
            if not torch.cuda.is_available():
                raise RuntimeError("daxq converts weights with HIP kernels and found no ROCm device "
                                   f"(module is on {home}); there is no CPU implementation")
            w = w.to(torch.device("cuda", torch.cuda.current_device()))

        weight_post_process.to(w.device)
        weight_post_process(w)
        if weight_post_process.dtype in FP8_ALLOWED_DTYPES:
            from ..quantized.functional import quantize_to_fp8 as quantize_func
        elif weight_post_process.dtype == torch.int8:
            from ..quantized.functional import quantize_to_int8 as quantize_func
        else:
            raise NotImplementedError(f"Unsupported dtype {weight_post_process.dtype}")

        weight_scale = weight_post_process.calculate_qparams()
        if weight_scale is not None:
            if weight_scale.numel() > 1:
                assert mod.weight.shape[0] == weight_scale.numel()
                scale_arg = weight_scale.reshape(-1, 1)
            else:
                scale_arg = weight_scale.reshape(1)
            qweight = quantize_func(w, scale=scale_arg, dtype=weight_post_process.dtype)
            qlinear.qweight = qweight.to(home)
            qlinear.weight_scale.copy_(weight_scale.reshape(qlinear.weight_scale.shape))
        if qlinear.bias is not None:
            qlinear.bias.copy_(mod.bias)

        if not reserve_float_weight:  # release the float parameters' memory
            del mod.weight
            del mod.bias
        qlinear.refresh_derived()
        return qlinear

    @classmethod
    def from_float(cls, mod, reserve_float_weight=False):
        if hasattr(mod, "weight_fake_quant"):  # QAT module carrying its own observers
            assert hasattr(mod, "activation_post_process"), "Input QAT module must have observer attached"
            weight_post_process = mod.weight_fake_quant
            activation_post_process = mod.activation_post_process
        else:
            assert type(mod) == cls._FLOAT_MODULE, (
                f" nnq.{cls.__name__}.from_float only works for {cls._FLOAT_MODULE.__name__} but got:{type(mod)}")
            assert hasattr(mod, "qconfig"), "Input float module must have qconfig defined."
            activation_post_process = mod.qconfig.activation()
            weight_post_process = mod.qconfig.weight()
        return cls.get_qlinear(mod, activation_post_process, weight_post_process, reserve_float_weight)
