"""The call that swaps a Wan2.1 transformer's linears for W8A8 ones.

``quantize_transformer`` is dax/adapters/wan/transformer_adapter.py:227-234: every ``nn.Linear``
of the DiT is quantised (per-token INT8 activations, per-channel INT8 weights) except the
``condition_embedder`` and ``proj_out`` subtrees.  ``fp8=True`` selects the e4m3fn pair the
reference documents in docs/linear_quantization.md:16-22.
"""
import torch

from ...quant.quantization import quantize_dynamic
from ...quant.quantization.qconfig import (
    get_dynamic_fp8_per_token_act_per_channel_weight_qconfig,
    get_dynamic_int8_per_token_act_per_channel_weight_qconfig,
)


def quantize_transformer(transformer, fp8: bool = False, fuse_blocks: bool = False):
    """``fuse_blocks`` additionally applies block_fusion.fuse_transformer_blocks (one quantisation per
    produced activation; takes the place of what the reference gets from torch.compile)."""
    if fp8:
        root = get_dynamic_fp8_per_token_act_per_channel_weight_qconfig(
            activation_dtype=torch.float8_e4m3fn, weight_dtype=torch.float8_e4m3fn)
    else:
        root = get_dynamic_int8_per_token_act_per_channel_weight_qconfig()
    qconfig_dict = {
        "": root,
        "condition_embedder": None,
        "proj_out": None,
    }
    quantize_dynamic(transformer, qconfig_dict)
    if fuse_blocks:
        from .block_fusion import fuse_transformer_blocks

        fuse_transformer_blocks(transformer)
