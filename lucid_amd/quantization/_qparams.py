"""``(scale, zero_point)`` from an observed range - on the device.

Mirrors ``lucid/quantization/_qparams.py:22-215`` (``QParams`` bundle and
``calculate_qparams``).  The reduction runs as one small HIP kernel
(``lq_calc_qparams``) so a dynamic-quantized layer never synchronises with the
host between the min/max reduction and the quantize kernel.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np

from .. import _C
from .._tensor import Tensor, float32, tensor
from ._qscheme import QDtype, QScheme


@dataclass(frozen=True)
class QParams:
    """Frozen bundle of quantization parameters (``_qparams.py:22-90``)."""

    scale: Tensor
    zero_point: Tensor
    qscheme: QScheme
    qdtype: QDtype
    ch_axis: int | None = None


def _as_hip_f32(v) -> Tensor:
    if isinstance(v, Tensor):
        if v.dtype != float32:
            raise _C.DtypeMismatch(f"calculate_qparams expects float32 ranges, got {v.dtype}")
        return v.to("hip")
    return tensor(np.float32(float(v)), device="hip")


def calculate_qparams(
    min_val, max_val, qscheme: QScheme, qdtype: QDtype, eps: float = 1e-8
) -> tuple[Tensor, Tensor]:
    """Derive ``(scale, zero_point)`` from an observed ``[min, max]`` range.

    Same arithmetic, in float32, as ``_qparams.py:198-215``: the range is first
    widened to contain 0; symmetric uses ``max|.| / ((qmax-qmin)/2)``, affine
    ``(max-min)/(qmax-qmin)`` and ``zp = clip(qmin - round(min/scale))``.
    """
    mn, mx = _as_hip_f32(min_val), _as_hip_f32(max_val)
    if mn.shape != mx.shape:
        raise _C.ShapeMismatch(f"min {mn.shape} and max {mx.shape} differ in shape")
    scale = Tensor.empty(mn.shape, float32, "hip")
    zp = Tensor.empty(mn.shape, float32, "hip")
    _C.call("lq_calc_qparams", mn.data_ptr, mx.data_ptr, mn.numel, int(qscheme.is_symmetric),
            qdtype.quant_min, qdtype.quant_max, int(qdtype.signed), float(eps), scale.data_ptr,
            zp.data_ptr, None)
    return scale, zp
