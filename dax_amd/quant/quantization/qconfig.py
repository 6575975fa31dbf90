"""QConfig factories for the dynamic W8A8 linear.

``get_dynamic_int8_per_token_act_per_channel_weight_qconfig`` and
``get_dynamic_fp8_per_token_act_per_channel_weight_qconfig`` have the names, arguments and
defaults of dax/quant/quantization/qconfig.py:157-179 and :85-107.  Note the FP8 default
activation dtype is ``float8_e5m2`` there; the gfx950 kernels implement e4m3fn, so pass
``activation_dtype=torch.float8_e4m3fn`` (an e5m2 config is reported as not implemented at
conversion and the layer stays in float, as the reference does for unsupported combinations).
"""
from collections import namedtuple

import torch

from ..qscheme import per_channel_symmetric, per_token_symmetric
from .observer import DynamicObserverPlaceholder, PerChannelMinMaxObserver

# activation / weight are observer factories (called with no arguments at conversion)
QConfig = namedtuple("QConfig", ["activation", "weight"])


def get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(
    activation_dtype=torch.float8_e5m2, weight_dtype=torch.float8_e4m3fn
):
    return QConfig(
        activation=DynamicObserverPlaceholder.with_args(
            dtype=activation_dtype, qscheme=per_token_symmetric, is_dynamic=True),
        weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric),
    )


def get_dynamic_int8_per_token_act_per_channel_weight_qconfig(
    activation_dtype=torch.int8, weight_dtype=torch.int8
):
    return QConfig(
        activation=DynamicObserverPlaceholder.with_args(
            dtype=activation_dtype, qscheme=per_token_symmetric, is_dynamic=True),
        weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric),
    )
