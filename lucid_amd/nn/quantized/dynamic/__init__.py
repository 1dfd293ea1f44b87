"""``lucid.nn.quantized.dynamic`` (``lucid/nn/quantized/dynamic/__init__.py``)."""

from .linear import Linear
from .rnn import LSTM

__all__ = ["Linear", "LSTM"]
