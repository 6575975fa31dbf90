from .linear import Linear, QuantizedActivation  # noqa: F401
