"""Range observers on the ``hip`` device.

Mirrors the observers the inference path uses
(``lucid/quantization/observer.py``): ``MinMaxObserver`` (:353-375),
``PerChannelMinMaxObserver`` (:623-653) and ``FixedQParamsObserver``
(:1113-1132) - same constructor arguments and defaults, buffers ``min_val`` /
``max_val`` seeded with +inf / -inf, ``with_args`` recipe helper (:239-247).
The statistics are one ``lq_minmax`` pass plus a fold kernel; nothing comes
back to the host.
"""

from __future__ import annotations

import functools

import numpy as np

from .. import _C
from .. import _tensor as T
from .._tensor import Tensor
from ..nn.module import Module
from ._functional import minmax
from ._qparams import calculate_qparams
from ._qscheme import (QDtype, QScheme, per_channel_symmetric, per_tensor_affine, qint8, quint8)


class ObserverBase(Module):
    def __init__(self, qscheme: QScheme, qdtype: QDtype, ch_axis: int | None, eps: float) -> None:
        super().__init__()
        self.qscheme, self.qdtype, self.ch_axis, self.eps = qscheme, qdtype, ch_axis, eps

    def calculate_qparams(self) -> tuple[Tensor, Tensor]:
        raise NotImplementedError

    @classmethod
    def with_args(cls, **kwargs):
        return functools.partial(cls, **kwargs)

    def _fold(self, cur_min: Tensor, cur_max: Tensor) -> None:
        run_min, run_max = self.min_val.to("hip"), self.max_val.to("hip")
        Cn = cur_min.numel
        scalar_seed = int(run_min.numel == 1 and Cn != 1)
        if not scalar_seed and run_min.numel != Cn:
            raise _C.ShapeMismatch(
                f"observer saw {Cn} channels after {run_min.numel}: the channel count changed")
        out_min = Tensor.empty(cur_min.shape, T.float32, "hip")
        out_max = Tensor.empty(cur_max.shape, T.float32, "hip")
        _C.call("lq_minmax_fold", run_min.data_ptr, run_max.data_ptr, cur_min.data_ptr,
                cur_max.data_ptr, Cn, scalar_seed, out_min.data_ptr, out_max.data_ptr, None)
        self.register_buffer("min_val", out_min)
        self.register_buffer("max_val", out_max)


class MinMaxObserver(ObserverBase):
    """Per-tensor running min / max (``observer.py:353-375``)."""

    def __init__(self, qscheme: QScheme = per_tensor_affine, qdtype: QDtype = quint8,
                 eps: float = 1e-8) -> None:
        super().__init__(qscheme, qdtype, None, eps)
        self.register_buffer("min_val", T.tensor(np.float32(np.inf)))
        self.register_buffer("max_val", T.tensor(np.float32(-np.inf)))

    def forward(self, x: Tensor) -> Tensor:
        mn, mx = minmax(x)
        self._fold(mn, mx)
        return x

    def calculate_qparams(self):
        return calculate_qparams(self.min_val, self.max_val, self.qscheme, self.qdtype, self.eps)


class PerChannelMinMaxObserver(ObserverBase):
    """Per-channel running min / max, reduced over all other axes
    (``observer.py:623-653``)."""

    def __init__(self, ch_axis: int = 0, qscheme: QScheme = per_channel_symmetric,
                 qdtype: QDtype = qint8, eps: float = 1e-8) -> None:
        super().__init__(qscheme, qdtype, ch_axis, eps)
        self.register_buffer("min_val", T.tensor(np.float32(np.inf)))
        self.register_buffer("max_val", T.tensor(np.float32(-np.inf)))

    def forward(self, x: Tensor) -> Tensor:
        axis = self.ch_axis if self.ch_axis is not None else 0
        mn, mx = minmax(x, ch_axis=axis)
        self._fold(mn, mx)
        return x

    def calculate_qparams(self):
        return calculate_qparams(self.min_val, self.max_val, self.qscheme, self.qdtype, self.eps)


class FixedQParamsObserver(ObserverBase):
    """Fixed ``(scale, zero_point)``; ``forward`` is the identity
    (``observer.py:1113-1132``)."""

    def __init__(self, scale: float, zero_point: int, qscheme: QScheme = per_tensor_affine,
                 qdtype: QDtype = quint8, eps: float = 1e-8) -> None:
        super().__init__(qscheme, qdtype, None, eps)
        self.register_buffer("scale", T.tensor(np.float32(float(scale))))
        self.register_buffer("zero_point", T.tensor(np.float32(float(zero_point))))

    def forward(self, x: Tensor) -> Tensor:
        return x

    def calculate_qparams(self):
        return self.scale, self.zero_point
