"""Stateful functional ops of a quantized graph - the residual joins
(``lucid/nn/quantized/functional_module.py:205-250``)."""

from __future__ import annotations

from ... import _C
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._qscheme import QDtype, quint8
from ..module import Module
from ._utils import activation_qparams, host_scalar, input_grid, storage_offset


class FloatFunctional(Module):
    """Calibration-time counterpart: ``prepare`` attaches an observer to it."""

    def add(self, x, y):
        raise NotImplementedError("float functional ops are outside the hip quantized path")

    add_relu = mul = add


class QFunctional(Module):
    def __init__(self, scale: Tensor, zero_point: Tensor, qdtype: QDtype = quint8) -> None:
        super().__init__()
        self.register_buffer("scale", scale.to("hip"))
        self.register_buffer("zero_point", zero_point.to("hip"))
        self.qdtype = qdtype
        self._zp_host = None

    def _state_loaded(self, name: str) -> None:
        if name == "zero_point":
            self._zp_host = None

    def _join(self, x: Tensor, y: Tensor, relu: bool) -> Tensor:
        gx, gy = input_grid(x, "QFunctional"), input_grid(y, "QFunctional")
        if x.shape != y.shape:
            raise _C.ShapeMismatch(f"QFunctional: shapes {x.shape} and {y.shape} differ")
        if gx.layout != gy.layout:
            raise _C.ShapeMismatch("QFunctional: operands are stored in different layouts")
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.qdtype)
        out = Tensor.empty(gx.codes.shape, T.int8, "hip")
        _C.call("lq_add_requant_i8", gx.codes.data_ptr, gx.offset, gx.scale.data_ptr,
                gx.zero_point.data_ptr, gy.codes.data_ptr, gy.offset, gy.scale.data_ptr,
                gy.zero_point.data_ptr, x.numel, int(relu), self.scale.data_ptr,
                self.zero_point.data_ptr, self.qdtype.quant_min, self.qdtype.quant_max, off,
                out.data_ptr, None)
        return Tensor.on_grid(x.shape, Grid(out, self.scale, self.zero_point, self.qdtype, off,
                                            self._zp_host, gx.layout))

    def add(self, x: Tensor, y: Tensor) -> Tensor:
        """Quantized ``x + y``."""
        return self._join(x, y, False)

    def add_relu(self, x: Tensor, y: Tensor) -> Tensor:
        """Quantized ``relu(x + y)``."""
        return self._join(x, y, True)

    @classmethod
    def from_float(cls, mod) -> "QFunctional":
        scale, zero_point, qdtype = activation_qparams(mod)
        return cls(scale, zero_point, qdtype)
