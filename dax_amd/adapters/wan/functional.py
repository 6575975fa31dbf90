"""``optimize_pipe``: the switch a Wan pipeline script flips (dax/adapters/wan/functional.py:9-40).

Only the linear-quantisation switch is built here (``int8_linear``, plus ``fp8_linear`` for the
documented e4m3fn configuration).  The reference's other switches drive subsystems that are not
part of this package and must stay off.
"""
from .transformer_adapter import quantize_transformer


def optimize_pipe(pipe, sequence_parallel=False, compile=False, overlap_comm=False, int8_linear=False,
                  cache_strategy=None, fp8_linear=False, fuse_blocks=False, **cache_params):
    if sequence_parallel or compile or overlap_comm or cache_strategy is not None or cache_params:
        raise NotImplementedError(
            "dax_amd builds the quantised-linear path only: sequence_parallel, compile, overlap_comm and "
            "cache_strategy must be left off")
    if int8_linear and fp8_linear:
        raise ValueError("choose one of int8_linear and fp8_linear")
    if int8_linear or fp8_linear:
        quantize_transformer(pipe.transformer, fp8=fp8_linear, fuse_blocks=fuse_blocks)
    return pipe
