"""Range observers on the ``hip`` device.

Mirrors the observers the inference path uses
(``lucid/quantization/observer.py``): ``MinMaxObserver`` (:353-375),
``PerChannelMinMaxObserver`` (:623-653) and ``FixedQParamsObserver``
(:1113-1132) - same constructor arguments and defaults, buffers ``min_val`` /
``max_val`` seeded with +inf / -inf, ``with_args`` recipe helper (:239-247) -
and the calibration-side ones: ``MovingAverageMinMaxObserver`` (:479-506),
``MovingAveragePerChannelMinMaxObserver`` (:988-1018) and ``HistogramObserver``
(:773-895).  The min / max observers are one ``lq_minmax`` pass plus a fold
kernel and nothing comes back to the host; the histogram observer reads its
scalars back exactly where Lucid's does (``.item()`` / ``.tolist()``).
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

    def _ema(self, cur_min: Tensor, cur_max: Tensor, per_channel: bool) -> None:
        run_min, run_max = self.min_val.to("hip"), self.max_val.to("hip")
        Cn = cur_min.numel
        scalar_seed = int(run_min.numel == 1 and Cn != 1)
        if not scalar_seed and run_min.numel != Cn:
            raise _C.ShapeMismatch(
                f"observer saw {Cn} channels after {run_min.numel}: the channel count changed")
        out_min = Tensor.empty(cur_min.shape, T.float32, "hip")
        out_max = Tensor.empty(cur_max.shape, T.float32, "hip")
        _C.call("lq_minmax_ema", run_min.data_ptr, run_max.data_ptr, cur_min.data_ptr, cur_max.data_ptr, Cn,
                scalar_seed, int(per_channel), float(self.averaging_constant), out_min.data_ptr,
                out_max.data_ptr, None)
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


class MovingAverageMinMaxObserver(MinMaxObserver):
    """EMA of the per-batch min / max, seeded by the first batch
    (``observer.py:479-506``)."""

    def __init__(self, qscheme: QScheme = per_tensor_affine, qdtype: QDtype = quint8,
                 averaging_constant: float = 0.01, eps: float = 1e-8) -> None:
        super().__init__(qscheme, qdtype, eps)
        self.averaging_constant = averaging_constant

    def forward(self, x: Tensor) -> Tensor:
        mn, mx = minmax(x)
        self._ema(mn, mx, per_channel=False)
        return x


class MovingAveragePerChannelMinMaxObserver(PerChannelMinMaxObserver):
    """Per-channel EMA (``observer.py:988-1018``)."""

    def __init__(self, ch_axis: int = 0, qscheme: QScheme = per_channel_symmetric,
                 qdtype: QDtype = qint8, averaging_constant: float = 0.01, eps: float = 1e-8) -> None:
        super().__init__(ch_axis, qscheme, qdtype, eps)
        self.averaging_constant = averaging_constant

    def forward(self, x: Tensor) -> Tensor:
        axis = self.ch_axis if self.ch_axis is not None else 0
        mn, mx = minmax(x, ch_axis=axis)
        self._ema(mn, mx, per_channel=True)
        return x


def _quantile_from_hist(counts, centers, q):
    """Bin centre at cumulative mass fraction ``q`` (``observer.py:880-895``)."""
    total = sum(counts)
    if total <= 0:
        return centers[0]
    target = q * total
    acc = 0.0
    for c, n in zip(centers, counts):
        acc += n
        if acc >= target:
            return c
    return centers[-1]


class HistogramObserver(ObserverBase):
    """Running histogram + L2-optimal clip range (``observer.py:773-878``).  The
    histogram is built on the device (``lq_histc_f32``); the range bookkeeping,
    the re-binning onto a wider range and the clip search run on the host in the
    same arithmetic as Lucid's (python floats and float32 tensor steps)."""

    def __init__(self, bins: int = 2048, qscheme: QScheme = per_tensor_affine, qdtype: QDtype = quint8,
                 eps: float = 1e-8) -> None:
        super().__init__(qscheme, qdtype, None, eps)
        self.bins = bins
        self.register_buffer("min_val", T.tensor(np.float32(np.inf)))
        self.register_buffer("max_val", T.tensor(np.float32(-np.inf)))
        self.register_buffer("histogram", T.tensor(np.zeros(bins, np.float32)))

    def _histc(self, x: Tensor, lo: float, hi: float) -> np.ndarray:
        out = Tensor.empty((self.bins,), T.float32, "hip")
        _C.call("lq_histc_f32", x.data_ptr, x.numel, float(lo), float(hi), self.bins, out.data_ptr, None)
        return out.numpy()

    def _rebin(self, hist: np.ndarray, old_min, old_max, new_min, new_max) -> np.ndarray:
        # observer.py:786-816, float32 tensor steps with python-float scalars
        bins, f32 = self.bins, np.float32
        old_width = (old_max - old_min) / bins
        new_width = (new_max - new_min) / bins
        centers = f32(old_min) + (np.arange(bins).astype(f32) + f32(0.5)) * f32(old_width)
        raw = np.clip((centers - f32(new_min)) / f32(new_width), f32(0.0), f32(bins - 1)).astype(f32)
        dst = raw.astype(np.int64)
        out = np.zeros(bins, f32)
        np.add.at(out, dst, hist.astype(f32))  # in index order, as scatter_add walks it
        return out

    def forward(self, x: Tensor) -> Tensor:
        if not isinstance(x, Tensor) or x.device != "hip" or x.dtype != T.float32:
            raise _C.DeviceMismatch("HistogramObserver: input must be a float32 tensor on the 'hip' device")
        mn, mx = minmax(x)
        cur_min, cur_max = float(mn.item()), float(mx.item())
        old_min, old_max = float(self.min_val.item()), float(self.max_val.item())
        if old_min == float("inf"):
            new_min, new_max = cur_min, cur_max
            hist = self._histc(x, new_min, new_max)
        else:
            new_min, new_max = min(old_min, cur_min), max(old_max, cur_max)
            hist = self._histc(x, new_min, new_max)
            old = self.histogram.numpy()
            if new_min == old_min and new_max == old_max:
                hist = (hist + old).astype(np.float32)
            else:
                hist = (hist + self._rebin(old, old_min, old_max, new_min, new_max)).astype(np.float32)
        self.register_buffer("min_val", T.tensor(np.float32(new_min)))
        self.register_buffer("max_val", T.tensor(np.float32(new_max)))
        self.register_buffer("histogram", T.tensor(hist))
        return x

    def _search_clip_range(self) -> tuple[float, float]:
        # observer.py:840-870, python-float arithmetic
        lo, hi = float(self.min_val.item()), float(self.max_val.item())
        counts = [float(v) for v in self.histogram.numpy().tolist()]
        total = sum(counts)
        if total <= 0.0 or hi <= lo:
            return lo, hi
        bins = self.bins
        width = (hi - lo) / bins
        centers = [lo + (i + 0.5) * width for i in range(bins)]
        levels = self.qdtype.quant_max - self.qdtype.quant_min
        best_err, best = float("inf"), (lo, hi)
        for frac in (0.0, 1e-5, 1e-4, 1e-3, 5e-3, 1e-2):
            cmin = _quantile_from_hist(counts, centers, frac)
            cmax = _quantile_from_hist(counts, centers, 1.0 - frac)
            if cmax <= cmin:
                continue
            step = (cmax - cmin) / max(levels, 1)
            err = 0.0
            for c, n in zip(centers, counts):
                if n == 0.0:
                    continue
                cc = cmin if c < cmin else (cmax if c > cmax else c)
                err += n * ((c - cc) ** 2 + (step * step) / 12.0)
            if err < best_err:
                best_err, best = err, (cmin, cmax)
        return best

    def calculate_qparams(self):
        new_min, new_max = self._search_clip_range()
        return calculate_qparams(T.tensor(np.float32(new_min), device="hip"),
                                 T.tensor(np.float32(new_max), device="hip"), self.qscheme, self.qdtype,
                                 self.eps)


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
