"""``lucid.nn.quantized`` on the hip device - the inference-path subset
(``lucid/nn/quantized/__init__.py``)."""

from . import dynamic
from .functional_module import FloatFunctional, QFunctional
from .conv import Conv1d, Conv2d, Conv3d
from .conv_transpose import ConvTranspose1d, ConvTranspose2d, ConvTranspose3d
from .intrinsic import ConvReLU1d, ConvReLU2d, ConvReLU3d, LinearReLU
from .linear import Linear
from .mlx_linear import QuantizedLinearMLX
from .modules import DeQuantize, DeQuantStub, Quantize, QuantStub, QuantWrapper
from .activation import ELU, Hardsigmoid, Hardswish, LeakyReLU, Sigmoid, Tanh
from .sparse import Embedding, EmbeddingBag

__all__ = ["QuantizedLinearMLX", "Linear", "LinearReLU", "Conv1d", "Conv2d", "Conv3d", "ConvReLU1d", "ConvReLU2d", "ConvReLU3d", "Quantize", "DeQuantize", "QuantStub", "DeQuantStub",
           "QuantWrapper", "QFunctional", "FloatFunctional", "dynamic", "Embedding", "EmbeddingBag", "ConvTranspose1d", "ConvTranspose2d", "ConvTranspose3d", "Sigmoid",
           "Hardswish", "Hardsigmoid", "Tanh", "ELU", "LeakyReLU"]
