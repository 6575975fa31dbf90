"""Which float module type is replaced by which quantised one (dax/quant/quantization/quantization_mappings.py:15-43)."""
import copy
from typing import Any, Callable, Dict, Set

from torch import nn

from ..nn import dynamic as nndq
from ..nn import quantized as nnsq

DEFAULT_STATIC_QUANT_MODULE_MAPPINGS: Dict[Callable, Any] = {
    nn.Linear: nnsq.Linear,
}

DEFAULT_DYNAMIC_QUANT_MODULE_MAPPINGS: Dict[Callable, Any] = {
    nn.Linear: nndq.Linear,
}


def get_default_qconfig_propagation_list() -> Set[Callable]:
    """Module types that get an observer in ``prepare`` (:26-33)."""
    return set(DEFAULT_STATIC_QUANT_MODULE_MAPPINGS.keys())


def get_default_static_quant_module_mappings() -> Dict[Callable, Any]:
    return copy.deepcopy(DEFAULT_STATIC_QUANT_MODULE_MAPPINGS)


def get_default_dynamic_quant_module_mappings() -> Dict[Callable, Any]:
    return copy.deepcopy(DEFAULT_DYNAMIC_QUANT_MODULE_MAPPINGS)
