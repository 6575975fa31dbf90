"""Pre-quantised checkpoints: save a quantised model once, load it without ever holding float weights.

The stored form is the module state the reference defines (dax/quant/nn/dynamic/linear.py:100-130:
``qweight`` [N, K] int8 / float8_e4m3fn, ``weight_scale`` fp32, ``bias`` bf16; the static module adds
``input_scale``, dax/quant/nn/quantized/linear.py:49-80).  That layout is also what the gfx950 GEMM
reads (K-contiguous rows are the MFMA operand order), so there is no separate packed format and
loading is a plain copy.

``load_quantized`` builds the quantised modules directly from the qconfig -- the same resolution rules
as ``quantize_dynamic`` (dax/quant/quantization/quantize.py:67-93) -- on a model whose float linears may
live on the ``meta`` device: a 14B transformer is brought up from an 8-bit file without a bf16 copy of
its linears ever existing.  The file format is safetensors (fp8 tensors are stored natively).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch
from torch import nn

from .nn import dynamic as nndq
from .quantization.quantize import _remove_qconfig, propagate_qconfig_


def save_quantized(model: nn.Module, path: str, metadata: Optional[Dict[str, str]] = None) -> None:
    """Writes ``model.state_dict()`` (quantised linears included) to a safetensors file."""
    from safetensors.torch import save_file

    state = {k: v.detach().contiguous().cpu() for k, v in model.state_dict().items()}
    save_file(state, path, metadata={"format": "daxq-w8a8", **(metadata or {})})


def _empty_quantised(mod: nn.Linear, device) -> nn.Module:
    act, wt = mod.qconfig.activation(), mod.qconfig.weight()
    if not getattr(act, "is_dynamic", False):
        from .nn.quantized import Linear as StaticLinear
        from .qscheme import per_channel_symmetric

        return StaticLinear(mod.in_features, mod.out_features, mod.bias is not None, device, wt.dtype, act.dtype,
                            mod.weight.dtype, wt.qscheme == per_channel_symmetric)
    return nndq.Linear(mod.in_features, mod.out_features, mod.bias is not None, device, wt.dtype, act.dtype,
                       mod.weight.dtype, wt.qscheme, act.qscheme)


def _swap_empty(module: nn.Module, device) -> None:
    for name, child in list(module.named_children()):
        _swap_empty(child, device)
        if type(child) is nn.Linear and getattr(child, "qconfig", None) is not None:
            module._modules[name] = _empty_quantised(child, device)


def load_quantized(model: nn.Module, path: str, qconfig_dict, device="cuda", strict: bool = True) -> nn.Module:
    """Turns ``model`` (float skeleton, parameters on any device including ``meta``) into its quantised
    form on ``device`` and fills it from the safetensors file at ``path``.  Every exact-type ``nn.Linear``
    whose resolved qconfig is not None becomes an (empty) quantised module first; no quantisation kernel
    runs and no float weight of those linears is read."""
    from safetensors.torch import load_file

    propagate_qconfig_(model, qconfig_dict)
    _swap_empty(model, torch.device(device))
    _remove_qconfig(model)
    # whatever is still on the meta device (unquantised layers of a meta skeleton) gets storage on `device`
    for mod in model.modules():
        for name, p in list(mod._parameters.items()):
            if p is not None and p.device.type == "meta":
                mod._parameters[name] = nn.Parameter(torch.empty_like(p, device=device), requires_grad=p.requires_grad)
        for name, b in list(mod._buffers.items()):
            if b is not None and b.device.type == "meta":
                mod._buffers[name] = torch.empty_like(b, device=device)
    model.to(device)
    state = load_file(path, device=str(device))
    model.load_state_dict(state, strict=strict)
    return model
