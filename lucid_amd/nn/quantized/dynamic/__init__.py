"""``lucid.nn.quantized.dynamic`` (``lucid/nn/quantized/dynamic/__init__.py``)."""

from .linear import Linear

__all__ = ["Linear"]
