"""``lucid.quantization`` on the ``hip`` device - the inference-path subset.

Names and signatures follow ``lucid/quantization/__init__.py:67-118``.
"""

from ._functional import dequantize, fake_quantize, minmax, quantize, quantize_rows_dynamic
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

from .observer import (FixedQParamsObserver, HistogramObserver, MinMaxObserver,
                       MovingAverageMinMaxObserver, MovingAveragePerChannelMinMaxObserver, ObserverBase,
                       PerChannelMinMaxObserver)
from .qconfig import QConfig, get_default_qat_qconfig, get_default_qconfig


def __getattr__(name):
    # the workflow functions import lucid_amd.nn, which imports this package
    if name == "FakeQuantize":
        from ._fake_quantize import FakeQuantize
        return FakeQuantize
    if name in ("prepare", "prepare_qat", "convert", "quantize_dynamic"):
        from . import _quantize
        return getattr(_quantize, name)
    if name in ("fuse_modules", "fuse_modules_qat"):
        from . import _fuse_modules
        return getattr(_fuse_modules, name)
    raise AttributeError(name)


__all__ = [
    "ObserverBase", "MinMaxObserver", "PerChannelMinMaxObserver", "FixedQParamsObserver",
    "MovingAverageMinMaxObserver", "MovingAveragePerChannelMinMaxObserver", "HistogramObserver",
    "QConfig", "get_default_qconfig", "prepare", "convert", "quantize_dynamic", "fuse_modules", "fuse_modules_qat",
    "QScheme", "per_tensor_affine", "per_tensor_symmetric", "per_channel_affine",
    "per_channel_symmetric", "QDtype", "qint8", "quint8", "qint32", "qint4", "QParams",
    "calculate_qparams", "quantize", "dequantize", "fake_quantize", "minmax", "quantize_rows_dynamic",
]
