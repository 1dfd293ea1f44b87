"""``QConfig``: an (activation observer recipe, weight observer recipe) pair
(``lucid/quantization/qconfig.py:35-190``)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from ._qscheme import per_channel_symmetric, per_tensor_affine, qint8, quint8
from .observer import MinMaxObserver, ObserverBase, PerChannelMinMaxObserver


@dataclass(frozen=True)
class QConfig:
    activation: Callable[[], ObserverBase]
    weight: Callable[[], ObserverBase]


def get_default_qconfig() -> QConfig:
    """quint8 affine activations, per-channel symmetric qint8 weights along
    axis 0.  Lucid's default activation observer is the histogram one
    (``qconfig.py``), which belongs to the calibration side that this backend
    does not rebuild; the min/max observer is used here."""
    return QConfig(
        activation=MinMaxObserver.with_args(qscheme=per_tensor_affine, qdtype=quint8),
        weight=PerChannelMinMaxObserver.with_args(ch_axis=0, qscheme=per_channel_symmetric,
                                                  qdtype=qint8),
    )
