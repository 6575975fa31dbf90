"""Module-swap machinery: resolve a qconfig for every submodule, then replace the mapped ones.

Same entry point and semantics as dax/quant/quantization/quantize.py:
``quantize_dynamic(model, qconfig_dict, mapping, inplace, remove_qconfig)`` (:394-444), and for the
static variant ``prepare`` (:250-301: attach an activation observer to every leaf module that is to be
quantised, called from a forward pre-hook) and ``convert`` (:360-391: swap by the static mapping).

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

from .quantization_mappings import (
    get_default_dynamic_quant_module_mappings,
    get_default_qconfig_propagation_list,
    get_default_static_quant_module_mappings,
)

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
        if pre_hook is not _observer_forward_pre_hook:  # the calibration observer goes away with the float module
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


def _observer_forward_pre_hook(self, input):
    """Shows the module's input to its activation observer (:28-31)."""
    self.activation_post_process(input[0])
    return None


def _remove_qconfig(module):
    """Drops qconfig attributes, activation observers and their hooks from the tree (:304-357)."""
    for child in module.children():
        _remove_qconfig(child)
    if hasattr(module, "qconfig"):
        del module.qconfig
    if "activation_post_process" in getattr(module, "_modules", {}):
        del module._modules["activation_post_process"]
    hooks = getattr(module, "_forward_pre_hooks", None)
    if hooks:
        for key in [k for k, fn in hooks.items() if fn is _observer_forward_pre_hook]:
            hooks.pop(key)


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


def _insert_activation_observer(module, device):
    """Adds ``activation_post_process`` to `module` and the pre-hook that shows it the module's input (:173-189)."""
    if getattr(module, "qconfig", None) is None:
        return
    observer = module.qconfig.activation()
    if device is not None:
        observer.to(device)
    module.add_module("activation_post_process", observer)
    module.register_forward_pre_hook(_observer_forward_pre_hook, prepend=True)


def _add_observer_(module, qconfig_propagation_list, non_leaf_module_list=None, device=None):
    """Gives every leaf module of a listed type with a qconfig an ``activation_post_process`` observer on
    the module's device, called first among its forward pre-hooks; a child whose type is in
    ``non_leaf_module_list`` gets one as a whole and is not descended into (:123-247)."""
    if device is None:
        devices = _module_devices(module)
        assert len(devices) <= 1, f"_add_observer_ only works with cpu or single-device CUDA modules, but got devices {devices}"
        device = next(iter(devices)) if devices else None
    for child in module.children():
        if type_before_parametrizations(child) is nn.Dropout:
            continue
        if non_leaf_module_list is not None and type_before_parametrizations(child) in non_leaf_module_list:
            _insert_activation_observer(child, device)
        else:
            _add_observer_(child, qconfig_propagation_list, non_leaf_module_list, device)
    is_leaf = not any(True for _ in module.children())
    if is_leaf and not isinstance(module, nn.Sequential) and type_before_parametrizations(module) in qconfig_propagation_list:
        _insert_activation_observer(module, device)


def prepare(model, qconfig_dict=None, inplace=True, observer_non_leaf_module_list=None):
    """Attaches qconfigs and activation observers for calibration (:250-301); run data through the model
    afterwards, then ``convert``."""
    if not inplace:
        model = copy.deepcopy(model)
    propagate_qconfig_(model, qconfig_dict)
    if not any(getattr(m, "qconfig", None) for m in model.modules()):
        import warnings

        warnings.warn("None of the submodule got qconfig applied. Make sure you passed correct configuration through "
                      "`qconfig_dict` or by assigning the `.qconfig` attribute directly on submodules")
    _add_observer_(model, get_default_qconfig_propagation_list(), observer_non_leaf_module_list)
    return model


def convert(model, mapping=None, inplace=True, remove_qconfig=True):
    """Swaps the prepared (and calibrated) modules by the static mapping (:360-391)."""
    if mapping is None:
        mapping = get_default_static_quant_module_mappings()
    if not inplace:
        model = copy.deepcopy(model)
    _convert(model, mapping)
    if remove_qconfig:
        _remove_qconfig(model)
    return model
