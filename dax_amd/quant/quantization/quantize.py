"""Module-swap machinery: resolve a qconfig for every submodule, then replace the mapped ones.

Same entry point and semantics as dax/quant/quantization/quantize.py:
``quantize_dynamic(model, qconfig_dict, mapping, inplace, remove_qconfig)`` (:394-444).

qconfig resolution per module (:67-93): a key equal to the module's *type* wins over what the
parent resolved to; a key equal to the module's dotted *name* ("" is the root) wins over that;
a ``qconfig`` attribute already on the module wins over both.  Children inherit the result, so
``{"": cfg, "proj_out": None}`` quantises everything except the ``proj_out`` subtree.
A module is swapped when its resolved qconfig is not None and its exact type is a key of the
mapping (:473-508); forward hooks and pre-hooks move to the new module and it is placed on the
device the old one was on.
"""
from __future__ import annotations

import copy

from torch import nn
from torch.nn.utils.parametrize import type_before_parametrizations

from .quantization_mappings import get_default_dynamic_quant_module_mappings

_UNSET = object()


def _propagate_qconfig_helper(module, qconfig_dict, qconfig_parent=None, prefix=""):
    cfg = qconfig_dict.get(type_before_parametrizations(module), qconfig_parent)
    cfg = qconfig_dict.get(prefix, cfg)
    cfg = getattr(module, "qconfig", cfg)
    if cfg is not None and not (hasattr(cfg, "activation") and hasattr(cfg, "weight")):
        raise AssertionError(f"qconfig for '{prefix}' must provide activation and weight observer factories, got {cfg!r}")
    module.qconfig = cfg
    for name, child in module.named_children():
        _propagate_qconfig_helper(child, qconfig_dict, cfg, f"{prefix}.{name}" if prefix else name)


def propagate_qconfig_(module, qconfig_dict=None):
    """Attaches the resolved ``qconfig`` attribute to every module of the tree, in place (:96-120)."""
    _propagate_qconfig_helper(module, qconfig_dict or {})


def _module_devices(mod):
    return {p.device for p in mod.parameters()} | {b.device for b in mod.buffers()}


def swap_module(mod, mapping, reserve_float_weight=False):
    """Returns the quantised counterpart of `mod`, or `mod` itself when it is not to be swapped (:473-508)."""
    if getattr(mod, "qconfig", None) is None:
        return mod
    target = mapping.get(type_before_parametrizations(mod))
    if target is None:
        return mod
    devices = _module_devices(mod)  # before from_float frees the float parameters
    assert len(devices) <= 1, f"swap_module only works with cpu or single-device CUDA modules, but got devices {devices}"
    new_mod = target.from_float(mod, reserve_float_weight)
    if new_mod is mod:
        return mod
    for pre_hook in mod._forward_pre_hooks.values():
        new_mod.register_forward_pre_hook(pre_hook)
    for hook in mod._forward_hooks.values():
        new_mod.register_forward_hook(hook)
    if devices:
        new_mod.to(next(iter(devices)))
    return new_mod


def _convert(module, mapping):
    """Post-order walk that swaps children in place (:447-470)."""
    for name, child in list(module.named_children()):
        _convert(child, mapping)
        module._modules[name] = swap_module(child, mapping)
    return module


def _remove_qconfig(module):
    for child in module.children():
        _remove_qconfig(child)
    if hasattr(module, "qconfig"):
        del module.qconfig


def quantize_dynamic(model, qconfig_dict=None, mapping=None, inplace=True, remove_qconfig=True):
    """Replaces the mapped float modules of `model` by dynamically quantised ones and returns the model."""
    if mapping is None:
        mapping = get_default_dynamic_quant_module_mappings()
    if not inplace:
        model = copy.deepcopy(model)
    propagate_qconfig_(model, qconfig_dict)
    _convert(model, mapping)
    if remove_qconfig:
        _remove_qconfig(model)
    return model


def prepare(model, *args, **kwargs):
    """Static-calibration entry point of the reference (:250-301); not part of the dynamic W8A8 path."""
    raise NotImplementedError("static calibration (prepare/convert) is not built; use quantize_dynamic")


def convert(model, *args, **kwargs):
    """Static-calibration entry point of the reference (:360-391); not part of the dynamic W8A8 path."""
    raise NotImplementedError("static calibration (prepare/convert) is not built; use quantize_dynamic")
