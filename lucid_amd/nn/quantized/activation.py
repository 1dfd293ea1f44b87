"""Quantized activations (``lucid/nn/quantized/activation.py:22-486``): the float
activation followed by a fake-quantize to the calibrated output grid.

An input that is carried as codes takes at most 256 values, so on codes the layer is a
256-entry table lookup built from exactly that formulation
(``requantize(act(dequantize(code)))``); a plain float input runs the float kernel with
the fake-quantize fused.
"""

from __future__ import annotations

from ... import _C
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._qscheme import QDtype, quint8
from ..module import Module
from ._utils import activation_qparams, host_scalar, storage_offset


def apply_activation(kind: int, alpha: float, x: Tensor, out_grid) -> Tensor:
    """``act(x)`` in float32; ``out_grid = (scale, zero_point, qdtype)`` adds the
    fake-quantize of ``activation.py:44-53``."""
    if not isinstance(x, Tensor) or x.device != "hip":
        raise _C.DeviceMismatch("activation: input must be a tensor on the 'hip' device")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"activation expects float32, got {x.dtype}")
    out = Tensor.empty(x.shape, T.float32, "hip")
    if out_grid is None:
        _C.call("lq_act_f32", kind, float(alpha), x.data_ptr, out.data_ptr, x.numel, 0, None, None, 0, 0, None)
    else:
        scale, zero_point, qdtype = out_grid
        _C.call("lq_act_f32", kind, float(alpha), x.data_ptr, out.data_ptr, x.numel, 1, scale.data_ptr,
                zero_point.data_ptr, qdtype.quant_min, qdtype.quant_max, None)
    return out


class _QuantizedActivation(Module):
    _kind = -1

    def __init__(self, scale: Tensor, zero_point: Tensor, qdtype: QDtype = quint8) -> None:
        super().__init__()
        self.register_buffer("scale", scale.to("hip"))
        self.register_buffer("zero_point", zero_point.to("hip"))
        self.qdtype = qdtype
        self._zp_host = None

    def _state_loaded(self, name: str) -> None:
        if name == "zero_point":
            self._zp_host = None

    def _alpha(self) -> float:
        return 0.0

    def _configure(self, mod) -> None:
        """Copy activation-specific parameters from the float module."""

    def forward(self, x: Tensor) -> Tensor:
        if not isinstance(x, Tensor) or x.device != "hip":
            raise _C.DeviceMismatch(f"{type(self).__name__}: input must be a tensor on the 'hip' device")
        if x._grid is None:
            return apply_activation(self._kind, self._alpha(), x, (self.scale, self.zero_point, self.qdtype))
        g = x._grid
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.qdtype)
        out = Tensor.empty(g.codes.shape, T.int8, "hip")
        _C.call("lq_act_requant_i8", self._kind, float(self._alpha()), g.codes.data_ptr, g.offset,
                g.scale.data_ptr, g.zero_point.data_ptr, g.codes.numel, self.scale.data_ptr,
                self.zero_point.data_ptr, self.qdtype.quant_min, self.qdtype.quant_max, off, out.data_ptr, None)
        return Tensor.on_grid(x.shape, Grid(out, self.scale, self.zero_point, self.qdtype, off, self._zp_host,
                                            g.layout))

    @classmethod
    def from_float(cls, mod):
        scale, zero_point, qdtype = activation_qparams(mod)
        obj = cls(scale, zero_point, qdtype)
        obj._configure(mod)
        return obj


class Sigmoid(_QuantizedActivation):
    _kind = 0


class Hardswish(_QuantizedActivation):
    _kind = 1


class Hardsigmoid(_QuantizedActivation):
    _kind = 2


class Tanh(_QuantizedActivation):
    _kind = 3


class ELU(_QuantizedActivation):
    _kind = 4
    alpha = 1.0

    def _configure(self, mod) -> None:
        self.alpha = float(getattr(mod, "alpha", 1.0))

    def _alpha(self) -> float:
        return self.alpha


class LeakyReLU(_QuantizedActivation):
    _kind = 5
    negative_slope = 0.01

    def _configure(self, mod) -> None:
        self.negative_slope = float(getattr(mod, "negative_slope", 0.01))

    def _alpha(self) -> float:
        return self.negative_slope
