from . import dynamic, quantized  # noqa: F401
