from .functional import FP8_ALLOWED_DTYPES, quantize_to_fp8, quantize_to_int8  # noqa: F401
from .linear import Linear  # noqa: F401
