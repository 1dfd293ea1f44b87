"""``lucid.nn.qat`` on the hip device: the forward of the quantization-aware-training layers
(weights and outputs fake-quantized every call) and their conversion to int8 modules.
``Linear`` and ``LinearReLU`` (``lucid/nn/qat/linear.py``); no backward pass - training is
Lucid's own business."""

from .linear import Linear, LinearReLU

__all__ = ["Linear", "LinearReLU"]
