"""``lucid.nn.quantized`` on the hip device - the inference-path subset
(``lucid/nn/quantized/__init__.py``)."""

from . import dynamic
from .functional_module import FloatFunctional, QFunctional
from .intrinsic import LinearReLU
from .linear import Linear
from .modules import DeQuantize, DeQuantStub, Quantize, QuantStub, QuantWrapper

__all__ = ["Linear", "LinearReLU", "Quantize", "DeQuantize", "QuantStub", "DeQuantStub",
           "QuantWrapper", "QFunctional", "FloatFunctional", "dynamic"]
