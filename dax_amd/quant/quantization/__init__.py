from .quantize import convert, prepare, quantize_dynamic  # noqa: F401
