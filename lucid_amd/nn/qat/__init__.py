"""``lucid.nn.qat`` on the hip device: the forward of the quantization-aware-training layers
(weights and outputs fake-quantized every call) and their conversion to int8 modules.
``Linear`` / ``LinearReLU`` (``lucid/nn/qat/linear.py``) and ``Conv2d`` / ``ConvReLU2d``
(``lucid/nn/qat/conv.py``); no backward pass - training is Lucid's own business."""

from .conv import Conv2d, ConvReLU2d
from .linear import Linear, LinearReLU

__all__ = ["Linear", "LinearReLU", "Conv2d", "ConvReLU2d"]
