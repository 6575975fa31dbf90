"""Static FP8 ``Linear``: calibrated per-tensor activation scale, per-tensor or per-channel weight.

Drop-in for dax/quant/nn/quantized/linear.py:28-251 -- same constructor signature and state
(``qweight`` parameter [N, K] in the fp8 weight dtype, ``weight_scale`` fp32 [1] or [1, N],
``input_scale`` fp32 [1], ``bias``), the same ``from_float`` / ``get_qlinear`` / ``weight`` /
``extra_repr`` surface.  ``forward`` (:91-118) is the leaf quantiser with the stored input scale
followed by the same MFMA GEMM as the dynamic module; the scalar scales are written out as the
per-row / per-channel vectors that kernel reads, which leaves the arithmetic per element unchanged:
``bf16((sum_k a*b) * input_scale * weight_scale + bias)``.

A pre-quantised checkpoint is loaded the way the reference does it: convert an uncalibrated model
(observers that have seen nothing give no scales, :170-176) and ``load_state_dict`` into it.
"""
from __future__ import annotations

import warnings

import torch
from torch import Tensor, nn

from .... import ops
from ...qscheme import per_channel_symmetric
from .._derived import DerivedOperands
from .functional import FP8_ALLOWED_DTYPES, quantize_to_fp8


class Linear(DerivedOperands, nn.Module):
    _FLOAT_MODULE = nn.Linear

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, weight_dtype=None,
                 input_dtype=None, out_dtype=None, row_wise_scale=False) -> None:
        if weight_dtype is not None and weight_dtype not in FP8_ALLOWED_DTYPES:
            raise NotImplementedError(f"the static linear is an FP8 module, got weight dtype {weight_dtype}")
        if input_dtype is not None and input_dtype not in FP8_ALLOWED_DTYPES:
            raise NotImplementedError(f"the static linear is an FP8 module, got input dtype {input_dtype}")
        if out_dtype not in (None, torch.bfloat16, torch.float16, torch.float32):
            raise NotImplementedError(f"daxq kernels produce bfloat16, float16 or float32 outputs, got out_dtype={out_dtype}")
        out_dtype = out_dtype if out_dtype is not None else torch.bfloat16
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.qweight = nn.Parameter(
            torch.empty((out_features, in_features), device=device, dtype=weight_dtype or torch.float8_e4m3fn),
            requires_grad=False)
        if bias:
            # the row-wise matmul writes bf16 and takes a bf16 bias whatever the module's dtype (:57-66)
            self.bias = nn.Parameter(torch.empty(out_features, device=device,
                                                 dtype=torch.bfloat16 if row_wise_scale else out_dtype))
        else:
            self.register_parameter("bias", None)
        self.register_buffer(
            "weight_scale", torch.ones((1, out_features) if row_wise_scale else 1, device=device, dtype=torch.float32),
            persistent=True)
        self.register_buffer("input_scale", torch.tensor([1.0], device=device, dtype=torch.float32), persistent=True)
        self.out_dtype = out_dtype
        self.weight_dtype = weight_dtype or torch.float8_e4m3fn
        self.input_dtype = input_dtype or torch.float8_e4m3fn
        self.row_wise_scale = row_wise_scale
        self._init_derived()

    @property
    def weight(self):
        """De-quantised weight in out_dtype (:87-89)."""
        return self.qweight.to(self.out_dtype) * self.weight_scale.reshape(-1, 1).to(self.out_dtype)

    def forward(self, input: Tensor) -> Tensor:
        self._check_device(input.device)
        prev_dims = input.shape[:-1]
        flat = input.view(-1, self.in_features)
        if flat.stride(-1) != 1:
            flat = flat.contiguous()
        sx = ops.broadcast_f32(self.input_scale.reshape(1), flat.shape[0])
        bias = None if self.bias is None else self.bias.detach()  # inference-only kernels
        x_fmt, w_fmt = ops.FMT_OF_DTYPE[self.input_dtype], ops.FMT_OF_DTYPE[self.weight_dtype]
        xq = getattr(ops, "quantize_rows_" + x_fmt)(flat, sx, True)
        # row-wise weight scales: the matmul writes bf16 and the result is cast afterwards (:96-104, :116-117)
        mm_dtype = torch.bfloat16 if self.row_wise_scale else self.out_dtype
        out = ops.linear_w8a8(xq, sx, self._gemm_weight(), self._weight_scale_vector(), bias, x_fmt, w_fmt, mm_dtype)
        out = out.view(*prev_dims, self.out_features)
        if out.dtype != self.out_dtype:
            out = out.to(self.out_dtype)
        return out

    def extra_repr(self) -> str:
        s = f"in_features={self.in_features}, out_features={self.out_features}"
        if self.bias is None:
            s += ", bias=False"
        s += f", weight_scale={self.weight_scale}, input_scale={self.input_scale}"
        return s

    @classmethod
    @torch.no_grad()
    def get_qlinear(cls, mod, activation_post_process, weight_post_process, reserve_float_weight):
        """Builds the static module from a float ``nn.Linear`` and its observers (:132-214).  With a
        calibrated activation observer the weight is observed and quantised too; without one (nothing
        observed) scales and quantised weight are left for a checkpoint to fill."""
        if activation_post_process is None or activation_post_process.dtype == torch.float:
            raise ValueError("Input must be quantized!")
        try:
            qlinear = cls(mod.in_features, mod.out_features, mod.bias is not None, mod.weight.device,
                          weight_post_process.dtype, activation_post_process.dtype, mod.weight.dtype,
                          weight_post_process.qscheme == per_channel_symmetric)
        except NotImplementedError as e:
            warnings.warn("Quantized linear is not supported for this combination of arguments. "
                          f"Falling back to float module. Message: {e}")
            return mod

        input_scale = activation_post_process.calculate_qparams()
        if input_scale is not None:
            qlinear.input_scale.copy_(input_scale.reshape(qlinear.input_scale.shape))
            home = mod.weight.device
            w = mod.weight.detach()
            if home.type != "cuda":
                if not torch.cuda.is_available():
                    raise RuntimeError("daxq converts weights with HIP kernels and found no ROCm device "
                                       f"(module is on {home}); there is no CPU implementation")
                w = w.to(torch.device("cuda", torch.cuda.current_device()))
            weight_post_process.to(w.device)
            weight_post_process(w)
            weight_scale = weight_post_process.calculate_qparams()
            if weight_scale is not None:
                if weight_scale.numel() > 1:
                    assert mod.weight.shape[0] == weight_scale.numel()
                    scale_arg = weight_scale.reshape(-1, 1)
                else:
                    scale_arg = weight_scale.reshape(1)
                qweight = quantize_to_fp8(w, scale=scale_arg, dtype=weight_post_process.dtype)
                qlinear.qweight = nn.Parameter(qweight.to(home), requires_grad=False)
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
            activation_post_process = getattr(mod, "activation_post_process", None)
            weight_post_process = mod.qconfig.weight()
        return cls.get_qlinear(mod, activation_post_process, weight_post_process, reserve_float_weight)
