"""``lucid.quantization`` on the ``hip`` device - the inference-path subset.

Names and signatures follow ``lucid/quantization/__init__.py:67-118``.
"""

from ._functional import dequantize, fake_quantize, minmax, quantize
from ._qparams import QParams, calculate_qparams
from ._qscheme import (
    QDtype,
    QScheme,
    per_channel_affine,
    per_channel_symmetric,
    per_tensor_affine,
    per_tensor_symmetric,
    qint4,
    qint8,
    qint32,
    quint8,
)

__all__ = [
    "QScheme", "per_tensor_affine", "per_tensor_symmetric", "per_channel_affine",
    "per_channel_symmetric", "QDtype", "qint8", "quint8", "qint32", "qint4", "QParams",
    "calculate_qparams", "quantize", "dequantize", "fake_quantize", "minmax",
]
