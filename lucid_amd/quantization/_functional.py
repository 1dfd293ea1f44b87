"""quantize / dequantize / fake_quantize on the ``hip`` device.

Mirrors ``lucid/quantization/_functional.py:57-448`` - same names, argument
meaning, defaults and dtypes.  Where Lucid composes each op from five to seven
engine calls (div, round, add, clip, astype ...), each is ONE fused HIP kernel
here; the per-element arithmetic and its order are unchanged.
"""

from __future__ import annotations

import ctypes as C

import numpy as np

from .. import _C
from .. import _tensor as T
from .._tensor import Tensor
from ._qscheme import QDtype


def _extents(shape, ch_axis):
    """Split ``shape`` around ``ch_axis`` into (outer, C, inner) - the
    broadcast of ``_reshape_for_channel`` (``_functional.py:45-54``)."""
    if ch_axis is None:
        return 1, 1, int(np.prod(shape, dtype=np.int64))
    nd = len(shape)
    if not -nd <= ch_axis < nd:
        raise IndexError(f"ch_axis {ch_axis} out of range for rank {nd}")
    ch_axis %= nd
    outer = int(np.prod(shape[:ch_axis], dtype=np.int64))
    inner = int(np.prod(shape[ch_axis + 1:], dtype=np.int64))
    return outer, int(shape[ch_axis]), inner


class _QP:
    """Resolved qparams: device pointers, or one host pair for Python scalars."""

    def __init__(self, scale, zero_point, ch_axis, shape):
        s_is_t, z_is_t = isinstance(scale, Tensor), isinstance(zero_point, Tensor)
        self.keep = []
        per_channel = ch_axis is not None and s_is_t
        self.outer, self.C, self.inner = _extents(shape, ch_axis if per_channel else None)
        if not s_is_t and not z_is_t:
            # a Python-float scale is rounded to float32 before the division
            # (scalar promotion, lucid/_dispatch.py:126-189)
            self.s = (C.c_float * 1)(np.float32(float(scale)))
            self.z = (C.c_float * 1)(np.float32(float(zero_point)))
            self.sp, self.zp, self.on_host = C.addressof(self.s), C.addressof(self.z), 1
            return
        st = self._dev(scale)
        zt = self._dev(zero_point)
        if per_channel:
            if st.numel != self.C:
                raise _C.ShapeMismatch(
                    f"scale has {st.numel} entries but axis {ch_axis} has {self.C} channels")
            if zt.numel == 1 and self.C != 1:
                zt = self._dev(T.tensor(np.full(self.C, zt.item(), np.float32)))
            if zt.numel != self.C:
                raise _C.ShapeMismatch(
                    f"zero_point has {zt.numel} entries but axis {ch_axis} has {self.C} channels")
        else:
            if st.numel != 1 or zt.numel != 1:
                raise _C.ShapeMismatch(
                    "per-tensor quantization needs one-element scale / zero_point "
                    "(pass ch_axis for per-channel parameters)")
        self.sp, self.zp, self.on_host = st.data_ptr, zt.data_ptr, 0

    def _dev(self, v) -> Tensor:
        # qparams may have been calibrated elsewhere; the math runs where the
        # data lives (_functional.py:166-174)
        if not isinstance(v, Tensor):
            v = T.tensor(np.float32(float(v)))
        if v.dtype != T.float32:
            raise _C.DtypeMismatch(f"scale / zero_point must be float32, got {v.dtype}")
        v = v.to("hip")
        self.keep.append(v)
        return v


def _require_hip(t: Tensor, what: str) -> None:
    if not isinstance(t, Tensor):
        raise TypeError(f"{what} expects a Tensor, got {type(t).__name__}")
    if t.device != "hip":
        raise _C.DeviceMismatch(
            f"{what}: tensor is on {t.device!r}; this backend computes on 'hip' only "
            "(move it with .to('hip'))")


def quantize(x: Tensor, scale, zero_point, qdtype: QDtype, ch_axis: int | None = None) -> Tensor:
    """``clip(round(x / scale) + zero_point, qmin, qmax)`` cast to the storage
    dtype of ``qdtype`` (``_functional.py:164-182``)."""
    _require_hip(x, "quantize")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"quantize expects float32 input, got {x.dtype}")
    storage = T.as_dtype(qdtype.storage)
    if storage not in (T.int8, T.int16):
        raise NotImplementedError(f"quantize to {qdtype!r} (storage {storage.name}) is not on this path")
    qp = _QP(scale, zero_point, ch_axis, x.shape)
    q = Tensor.empty(x.shape, storage, "hip")
    _C.call("lq_quantize", x.data_ptr, q.data_ptr, storage.code, 0, qp.outer, qp.C, qp.inner,
            qp.sp, qp.zp, qp.on_host, qdtype.quant_min, qdtype.quant_max, None)
    return q


def dequantize(q: Tensor, scale, zero_point, ch_axis: int | None = None) -> Tensor:
    """``(q.to(float32) - zero_point) * scale`` (``_functional.py:269-281``)."""
    _require_hip(q, "dequantize")
    if q.dtype not in (T.int8, T.int16):
        raise _C.DtypeMismatch(f"dequantize expects int8 / int16 codes, got {q.dtype}")
    qp = _QP(scale, zero_point, ch_axis, q.shape)
    out = Tensor.empty(q.shape, T.float32, "hip")
    _C.call("lq_dequantize", q.data_ptr, q.dtype.code, 0, out.data_ptr, qp.outer, qp.C, qp.inner,
            qp.sp, qp.zp, qp.on_host, None)
    return out


def fake_quantize(x: Tensor, scale, zero_point, quant_min: int, quant_max: int,
                  ch_axis: int | None = None) -> Tensor:
    """``dequantize(quantize(x))`` kept in float32 (``_functional.py:299-313``).
    Forward only: this path is inference, so no straight-through mask is saved."""
    _require_hip(x, "fake_quantize")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"fake_quantize expects float32 input, got {x.dtype}")
    qp = _QP(scale, zero_point, ch_axis, x.shape)
    out = Tensor.empty(x.shape, T.float32, "hip")
    _C.call("lq_fake_quantize", x.data_ptr, out.data_ptr, qp.outer, qp.C, qp.inner, qp.sp, qp.zp,
            qp.on_host, int(quant_min), int(quant_max), None)
    return out


def quantize_rows_dynamic(x: Tensor, qscheme, qdtype: QDtype, eps: float = 1e-8
                          ) -> tuple[Tensor, Tensor, Tensor]:
    """Per-row ("per-token") dynamic quantization of a 2-d float32 tensor in one pass:
    ``(codes, scale, zero_point)`` equal, bit for bit, to

        mn, mx = minmax(x, ch_axis=0)
        scale, zero_point = calculate_qparams(mn, mx, qscheme, qdtype, eps)
        codes = quantize(x, scale, zero_point, qdtype, ch_axis=0)

    (``observer.py:634-653``, ``_qparams.py:198-215``, ``_functional.py:164-182``) with ``x``
    read once.  Rows the one-pass kernel does not take (longer than 16384, not a multiple
    of 4, int16 storage) go through those three calls."""
    from ._qparams import calculate_qparams
    _require_hip(x, "quantize_rows_dynamic")
    if x.dtype != T.float32 or x.ndim != 2:
        raise _C.DtypeMismatch(f"quantize_rows_dynamic expects a 2-d float32 tensor, got {x.dtype} {x.shape}")
    rows, cols = x.shape
    storage = T.as_dtype(qdtype.storage)
    if storage == T.int8 and cols % 4 == 0 and 4 <= cols <= 16384 and x.data_ptr % 16 == 0:
        q = Tensor.empty(x.shape, T.int8, "hip")
        scale = Tensor.empty((rows,), T.float32, "hip")
        zp = Tensor.empty((rows,), T.float32, "hip")
        _C.call("lq_quantize_rows_dynamic_i8", x.data_ptr, rows, cols, int(qscheme.is_symmetric),
                qdtype.quant_min, qdtype.quant_max, int(qdtype.signed), float(eps), 0, scale.data_ptr,
                zp.data_ptr, None, None, q.data_ptr, None)
        return q, scale, zp
    mn, mx = minmax(x, ch_axis=0)
    scale, zp = calculate_qparams(mn, mx, qscheme, qdtype, eps)
    return quantize(x, scale, zp, qdtype, ch_axis=0), scale, zp


def minmax(x: Tensor, ch_axis: int | None = None) -> tuple[Tensor, Tensor]:
    """Min and max of ``x`` in one pass: global (0-d results) or per channel
    along ``ch_axis`` (length-C results).  NaN-propagating, as Lucid's
    reductions are (``lucid/_C/backend/cpu/Reduce.cpp:87-125``)."""
    _require_hip(x, "minmax")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"minmax expects float32 input, got {x.dtype}")
    outer, Cn, inner = _extents(x.shape, ch_axis)
    shape = () if ch_axis is None else (Cn,)
    mn = Tensor.empty(shape, T.float32, "hip")
    mx = Tensor.empty(shape, T.float32, "hip")
    _C.call("lq_minmax", x.data_ptr if x.numel else None, outer, Cn, inner, mn.data_ptr,
            mx.data_ptr, None)
    return mn, mx
