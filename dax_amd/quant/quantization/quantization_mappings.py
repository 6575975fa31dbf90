"""Which float module type is replaced by which quantised one (dax/quant/quantization/quantization_mappings.py:21-43)."""
import copy
from typing import Any, Callable, Dict

from torch import nn

from ..nn import dynamic as nndq

DEFAULT_DYNAMIC_QUANT_MODULE_MAPPINGS: Dict[Callable, Any] = {
    nn.Linear: nndq.Linear,
}


def get_default_dynamic_quant_module_mappings() -> Dict[Callable, Any]:
    return copy.deepcopy(DEFAULT_DYNAMIC_QUANT_MODULE_MAPPINGS)
