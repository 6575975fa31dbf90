from .transformer_adapter import quantize_transformer  # noqa: F401
from .functional import optimize_pipe  # noqa: F401
