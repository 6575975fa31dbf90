"""Observers: what a qconfig instantiates to describe how a tensor is quantised.

Counterparts of dax/quant/quantization/observer.py.  Two are on the dynamic W8A8 path:

* ``PerChannelMinMaxObserver``  (:229-374) -- per-output-channel weight statistics; the row
  min / max and the scale ``max(max(-min, max) / qmax, eps)`` (:97-134, fp32 throughout) are
  computed by the HIP kernels ``daxq_row_minmax`` / ``daxq_scale_from_minmax``;
* ``DynamicObserverPlaceholder`` (:453-477) -- an inert carrier of dtype and qscheme for a
  dynamically quantised activation.

``MinMaxObserver`` (:141-226) is the per-tensor observer of the static and per-tensor variants:
running min / max of everything shown to it, reduced on the device (``daxq_row_minmax`` +
``daxq_tensor_minmax_update``).  The histogram profiler (``DistributionProfileObserver``, a
calibration diagnostic that writes plots) is not built.
"""
from __future__ import annotations

from functools import partial

import torch
from torch import nn

from ... import ops
from ..qscheme import per_channel_symmetric, per_tensor_symmetric, per_token_symmetric

ALLOWED_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2, torch.int8)


class UniformQuantizationObserverBase(nn.Module):
    """Holds dtype, qscheme, quant_max and the scale floor ``eps`` (:19-56)."""

    def __init__(self, dtype=torch.float8_e4m3fn, qscheme=per_tensor_symmetric, factory_kwargs=None,
                 eps=torch.finfo(torch.float32).eps, is_dynamic=False, prefix="", sync_state=False, **kwargs) -> None:
        super().__init__()
        assert qscheme in (per_tensor_symmetric, per_channel_symmetric, per_token_symmetric), (
            "Default Observer only works for per_tensor_symmetric/per_channel_symmetric/per_token_symmetric "
            "quantization scheme")
        assert dtype in ALLOWED_DTYPES, f"Default Observer only works for {ALLOWED_DTYPES} data type"
        self.dtype = dtype
        self.is_dynamic = is_dynamic
        self.qscheme = qscheme
        fk = factory_kwargs or {}
        self.register_buffer("eps", torch.tensor([eps], **fk))
        self.quant_max = torch.iinfo(dtype).max if dtype == torch.int8 else torch.finfo(dtype).max
        self.prefix = prefix
        self.sync_state = sync_state

    @classmethod
    def with_args(cls, **kwargs):
        """A factory that builds this observer with the given arguments (what QConfig stores)."""
        return partial(cls, **kwargs)

    def _calculate_qparams(self, min_val: torch.Tensor, max_val: torch.Tensor):
        if min_val.numel() == 0 or max_val.numel() == 0:
            return None  # nothing observed yet (:116-120)
        return ops.scale_from_minmax(min_val, max_val, float(self.quant_max), float(self.eps))

    def reset_min_max_vals(self):
        raise NotImplementedError("Cannot reset min/max values in the given observer.")


class MinMaxObserver(UniformQuantizationObserverBase):
    """Running per-tensor min / max (:141-226); ``calculate_qparams`` gives the fp32 scale [1] or None
    while nothing has been observed."""

    def __init__(self, dtype=torch.float8_e4m3fn, qscheme=per_tensor_symmetric, factory_kwargs=None,
                 eps=torch.finfo(torch.float32).eps, is_dynamic=False, **kwargs) -> None:
        assert qscheme == per_tensor_symmetric, "MinMaxObserver's qscheme only support per_tensor_symmetric"
        super().__init__(dtype=dtype, qscheme=qscheme, factory_kwargs=factory_kwargs, eps=eps,
                         is_dynamic=is_dynamic, **kwargs)
        fk = factory_kwargs or {}
        self.register_buffer("min_val", torch.tensor(float("inf"), **fk))
        self.register_buffer("max_val", torch.tensor(float("-inf"), **fk))

    def forward(self, x_orig):
        if x_orig.numel() == 0:
            return x_orig
        x = x_orig.detach()
        x = x.reshape(-1, x.shape[-1]) if x.dim() > 1 else x.reshape(1, -1)
        if x.stride(1) != 1:
            x = x.contiguous()
        lo, hi = ops.row_minmax(x)
        if self.min_val.device != lo.device:
            self.min_val = self.min_val.to(lo.device)
            self.max_val = self.max_val.to(lo.device)
        lo1, hi1 = self.min_val.reshape(1).clone(), self.max_val.reshape(1).clone()
        ops.tensor_minmax_update(lo, hi, lo1, hi1)
        self.min_val.copy_(lo1.reshape(()))
        self.max_val.copy_(hi1.reshape(()))
        self._sync_state()
        return x_orig

    def _sync_state(self):
        if self.sync_state and torch.distributed.is_available() and torch.distributed.is_initialized():
            raise NotImplementedError("daxq is built for one GPU: observers with sync_state=True cannot reduce over ranks")

    def calculate_qparams(self):
        lo, hi = self.min_val.reshape(1), self.max_val.reshape(1)
        if bool(lo == float("inf")) and bool(hi == float("-inf")):
            return None  # the untouched state: nothing observed yet, a pre-quantised checkpoint supplies the scales
        return self._calculate_qparams(lo, hi)  # a real +-inf in the calibration data gives an infinite scale, as there

    def extra_repr(self):
        return f"min_val={self.min_val}, max_val={self.max_val}"

    def reset_min_max_vals(self):
        self.min_val.fill_(float("inf"))
        self.max_val.fill_(float("-inf"))


class PerChannelMinMaxObserver(UniformQuantizationObserverBase):
    """Running per-channel min / max of everything it has been shown (:229-374)."""

    def __init__(self, ch_axis=0, dtype=torch.float8_e4m3fn, qscheme=per_tensor_symmetric, factory_kwargs=None,
                 eps=torch.finfo(torch.float32).eps, is_dynamic=False, **kwargs) -> None:
        if not qscheme == per_channel_symmetric:
            raise NotImplementedError("PerChannelMinMaxObserver's qscheme only support per_channel_symmetric,")
        super().__init__(dtype=dtype, qscheme=qscheme, factory_kwargs=factory_kwargs, eps=eps,
                         is_dynamic=is_dynamic, **kwargs)
        fk = factory_kwargs or {}
        self.ch_axis = ch_axis
        self.register_buffer("min_val", torch.tensor([], **fk))
        self.register_buffer("max_val", torch.tensor([], **fk))

    def forward(self, x_orig):
        if x_orig.numel() == 0:
            return x_orig
        x = x_orig.detach()
        if self.ch_axis != 0:
            x = x.transpose(0, self.ch_axis)
        x = x.reshape(x.shape[0], -1)
        if x.stride(1) != 1:
            x = x.contiguous()
        lo, hi = ops.row_minmax(x)
        if self.min_val.numel() != 0 and self.max_val.numel() != 0:
            lo = torch.minimum(lo, self.min_val.to(lo.device))
            hi = torch.maximum(hi, self.max_val.to(hi.device))
        self.min_val = lo
        self.max_val = hi
        return x_orig

    def calculate_qparams(self):
        return self._calculate_qparams(self.min_val, self.max_val)

    def extra_repr(self):
        return f"min_val={self.min_val}, max_val={self.max_val}"

    def reset_min_max_vals(self):
        self.min_val = torch.tensor([], device=self.min_val.device)
        self.max_val = torch.tensor([], device=self.max_val.device)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        # buffers start empty; size them to whatever the checkpoint holds (:336-374)
        for name in ("min_val", "max_val"):
            key = prefix + name
            if key in state_dict:
                setattr(self, name, torch.empty_like(state_dict[key], device=getattr(self, name).device))
            elif strict:
                missing_keys.append(key)
        super()._load_from_state_dict(state_dict, prefix, local_metadata, False, missing_keys, unexpected_keys,
                                      error_msgs)


class DynamicObserverPlaceholder(UniformQuantizationObserverBase):
    """Carries dtype / qscheme for an activation quantised at run time; observes nothing (:453-477)."""

    def forward(self, x_orig):
        pass

    def calculate_qparams(self):
        pass
