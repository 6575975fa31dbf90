"""QConfig factories: which observer describes the activation and which the weight.

Names, arguments and defaults of dax/quant/quantization/qconfig.py:13-212.  The two on the DiT hot
path are ``get_dynamic_int8_per_token_act_per_channel_weight_qconfig`` (:157-179) and
``get_dynamic_fp8_per_token_act_per_channel_weight_qconfig`` (:85-107; its default activation dtype
is ``float8_e5m2``, pass ``activation_dtype=torch.float8_e4m3fn`` for the e4m3fn pair).  The static
factories (:13-59) pair with ``prepare`` / ``convert``; the per-tensor dynamic ones (:61-83,
:109-155) with ``quantize_dynamic``.  FP8 weights are e4m3fn on gfx950; an e5m2 weight config is
reported as not implemented at conversion and the layer stays in float.
"""
from collections import namedtuple

import torch

from ..qscheme import per_channel_symmetric, per_tensor_symmetric, per_token_symmetric
from .observer import DynamicObserverPlaceholder, MinMaxObserver, PerChannelMinMaxObserver

# activation / weight are observer factories (called with no arguments at conversion)
QConfig = namedtuple("QConfig", ["activation", "weight"])


def _dynamic(dtype, qscheme):
    return DynamicObserverPlaceholder.with_args(dtype=dtype, qscheme=qscheme, is_dynamic=True)


# ------------------------------------------------------------------ static (calibrated activation scale)
def get_default_fp8_qconfig(activation_dtype=torch.float8_e5m2, weight_dtype=torch.float8_e4m3fn):
    """Per-tensor activation and weight, both from running min / max (:13-34)."""
    return QConfig(
        activation=MinMaxObserver.with_args(dtype=activation_dtype, qscheme=per_tensor_symmetric, sync_state=True),
        weight=MinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_tensor_symmetric))


def get_fp8_per_channel_weight_qconfig(activation_dtype=torch.float8_e5m2, weight_dtype=torch.float8_e4m3fn):
    """Per-tensor calibrated activation, per-channel weight (:37-58)."""
    return QConfig(
        activation=MinMaxObserver.with_args(dtype=activation_dtype, qscheme=per_tensor_symmetric, sync_state=True),
        weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric))


# ------------------------------------------------------------------ dynamic
def get_default_dynamic_fp8_qconfig(activation_dtype=torch.float8_e5m2, weight_dtype=torch.float8_e4m3fn):
    """Per-tensor dynamic activation, per-tensor weight (:61-82)."""
    return QConfig(activation=_dynamic(activation_dtype, per_tensor_symmetric),
                   weight=MinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_tensor_symmetric))


def get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(
    activation_dtype=torch.float8_e5m2, weight_dtype=torch.float8_e4m3fn
):
    return QConfig(activation=_dynamic(activation_dtype, per_token_symmetric),
                   weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric))


def get_default_dynamic_int8_qconfig(activation_dtype=torch.int8, weight_dtype=torch.int8):
    """Per-tensor dynamic activation, per-tensor weight (:109-130)."""
    return QConfig(activation=_dynamic(activation_dtype, per_tensor_symmetric),
                   weight=MinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_tensor_symmetric))


def get_dynamic_int8_per_channel_weight_qconfig(activation_dtype=torch.int8, weight_dtype=torch.int8):
    """Per-tensor dynamic activation, per-channel weight (:133-154)."""
    return QConfig(activation=_dynamic(activation_dtype, per_tensor_symmetric),
                   weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric))


def get_dynamic_int8_per_token_act_per_channel_weight_qconfig(
    activation_dtype=torch.int8, weight_dtype=torch.int8
):
    return QConfig(activation=_dynamic(activation_dtype, per_token_symmetric),
                   weight=PerChannelMinMaxObserver.with_args(dtype=weight_dtype, qscheme=per_channel_symmetric))


def get_default_dist_profile_qconfig(*args, **kwargs):
    """The reference's histogram profiler (:181-212) writes distribution plots during calibration; it
    computes nothing the quantised model uses and is not built."""
    raise NotImplementedError("the distribution-profile observer (a calibration diagnostic) is not part of daxq")
