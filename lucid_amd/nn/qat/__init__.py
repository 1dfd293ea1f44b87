"""``lucid.nn.qat`` on the hip device: the forward of the quantization-aware-training layers
(weights and outputs fake-quantized every call) and their conversion to int8 modules.
``Linear`` / ``LinearReLU`` (``lucid/nn/qat/linear.py``), ``Conv1d / 2d / 3d`` and
``ConvReLU1d / 2d / 3d`` (``lucid/nn/qat/conv.py``), ``Embedding`` (``lucid/nn/qat/sparse.py``);
no backward pass - training is Lucid's own business."""

from .conv import Conv1d, Conv2d, Conv3d, ConvReLU1d, ConvReLU2d, ConvReLU3d
from .linear import Linear, LinearReLU
from .sparse import Embedding

__all__ = ["Linear", "LinearReLU", "Conv1d", "Conv2d", "Conv3d", "ConvReLU1d", "ConvReLU2d", "ConvReLU3d",
           "Embedding"]
