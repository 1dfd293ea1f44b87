"""``QConfig``: an (activation observer recipe, weight observer recipe) pair
(``lucid/quantization/qconfig.py:35-190``)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from ._qscheme import per_channel_symmetric, per_tensor_affine, qint8, quint8
from .observer import (HistogramObserver, MovingAverageMinMaxObserver, ObserverBase,
                       PerChannelMinMaxObserver)


@dataclass(frozen=True)
class QConfig:
    activation: Callable[[], ObserverBase]
    weight: Callable[[], ObserverBase]


def get_default_qconfig() -> QConfig:
    """Histogram observer on quint8 affine activations, per-channel symmetric
    qint8 weights along axis 0 (``qconfig.py:150-190``)."""
    return QConfig(
        activation=HistogramObserver.with_args(qscheme=per_tensor_affine, qdtype=quint8),
        weight=PerChannelMinMaxObserver.with_args(ch_axis=0, qscheme=per_channel_symmetric,
                                                  qdtype=qint8),
    )


def get_default_qat_qconfig() -> QConfig:
    """The QAT recipe (``qconfig.py:193-258``): the same grids as the default PTQ config, each
    observer wrapped in a ``FakeQuantize`` - moving-average min/max on quint8 affine
    activations, per-channel symmetric qint8 weights along axis 0."""
    from ._fake_quantize import FakeQuantize
    return QConfig(
        activation=FakeQuantize.with_args(observer=MovingAverageMinMaxObserver, qscheme=per_tensor_affine,
                                          qdtype=quint8),
        weight=FakeQuantize.with_args(observer=PerChannelMinMaxObserver, ch_axis=0,
                                      qscheme=per_channel_symmetric, qdtype=qint8),
    )
