from .transformer_adapter import quantize_transformer  # noqa: F401
from .functional import optimize_pipe  # noqa: F401
from .block_fusion import fuse_linears, fuse_transformer_blocks, share_input_quant  # noqa: F401
