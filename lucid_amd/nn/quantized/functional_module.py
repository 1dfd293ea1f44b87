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

    def _out(self, shape, codes, layout) -> Tensor:
        return Tensor.on_grid(shape, Grid(codes, self.scale, self.zero_point, self.qdtype,
                                          storage_offset(self.qdtype), self._zp_host, layout))

    def _binary(self, op: int, x: Tensor, y, relu: bool = False) -> Tensor:
        """``fq(act(x OP y))``; ``y`` a tensor on a grid or a Python scalar."""
        gx = input_grid(x, "QFunctional")
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.qdtype)
        out = Tensor.empty(gx.codes.shape, T.int8, "hip")
        if isinstance(y, Tensor):
            gy = input_grid(y, "QFunctional")
            if x.shape != y.shape:
                raise _C.ShapeMismatch(f"QFunctional: shapes {x.shape} and {y.shape} differ")
            if gx.layout != gy.layout:
                raise _C.ShapeMismatch("QFunctional: operands are stored in different layouts")
            b = (gy.codes.data_ptr, gy.offset, gy.scale.data_ptr, gy.zero_point.data_ptr, 0.0)
        else:
            b = (None, 0, None, None, float(y))
        _C.call("lq_binary_requant_i8", op, gx.codes.data_ptr, gx.offset, gx.scale.data_ptr,
                gx.zero_point.data_ptr, *b, x.numel, int(relu), self.scale.data_ptr,
                self.zero_point.data_ptr, self.qdtype.quant_min, self.qdtype.quant_max, off, out.data_ptr,
                None)
        return self._out(x.shape, out, gx.layout)

    def add(self, x: Tensor, y: Tensor) -> Tensor:
        """Quantized ``x + y``."""
        return self._join(x, y, False)

    def mul(self, x: Tensor, y: Tensor) -> Tensor:
        """Quantized ``x * y``."""
        return self._binary(1, x, y)

    def add_scalar(self, x: Tensor, scalar: float) -> Tensor:
        """Quantized ``x + scalar``."""
        return self._binary(0, x, float(scalar))

    def mul_scalar(self, x: Tensor, scalar: float) -> Tensor:
        """Quantized ``x * scalar``."""
        return self._binary(1, x, float(scalar))

    def cat(self, tensors: list[Tensor], dim: int = 0) -> Tensor:
        """Quantized concatenation along ``dim`` (batch, or channels / features):
        each operand is re-expressed on this module's output grid."""
        if not tensors:
            raise ValueError("QFunctional.cat: nothing to concatenate")
        grids = [input_grid(t, "QFunctional") for t in tensors]
        layout, nd = grids[0].layout, tensors[0].ndim
        if any(g.layout != layout for g in grids) or any(t.ndim != nd for t in tensors):
            raise _C.ShapeMismatch("QFunctional.cat: operands differ in rank or storage layout")
        dim %= nd
        if dim not in (0, 1):
            raise NotImplementedError("QFunctional.cat on hip: dim 0 (batch) or 1 (channels / features)")
        for t in tensors:
            if any(a != b for i, (a, b) in enumerate(zip(t.shape, tensors[0].shape)) if i != dim):
                raise _C.ShapeMismatch("QFunctional.cat: operands differ outside the concatenated axis")
        if dim == 1 and layout == "plain" and nd > 2:
            raise NotImplementedError("QFunctional.cat on hip: channel concatenation needs NHWC or 2-d codes")
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.qdtype)
        total = sum(t.shape[dim] for t in tensors)
        shape = list(tensors[0].shape)
        shape[dim] = total
        # codes are stored [B, (H, W,) C] for nhwc and as the float shape otherwise
        cshape = list(grids[0].codes.shape)
        cshape[0 if dim == 0 else -1] = total
        out = Tensor.empty(tuple(cshape), T.int8, "hip")
        at = 0
        for t, g in zip(tensors, grids):
            if dim == 0:
                rows, cols, ld, dst = 1, g.codes.numel, g.codes.numel, out.data_ptr + at
                at += g.codes.numel
            else:
                cols = t.shape[1]
                rows, ld, dst = g.codes.numel // cols, total, out.data_ptr + at
                at += cols
            _C.call("lq_requant_rows_i8", g.codes.data_ptr, g.offset, g.scale.data_ptr, g.zero_point.data_ptr,
                    rows, cols, dst, ld, self.scale.data_ptr, self.zero_point.data_ptr, self.qdtype.quant_min,
                    self.qdtype.quant_max, off, None)
        return self._out(tuple(shape), out, layout)

    def add_relu(self, x: Tensor, y: Tensor) -> Tensor:
        """Quantized ``relu(x + y)``."""
        return self._join(x, y, True)

    @classmethod
    def from_float(cls, mod) -> "QFunctional":
        scale, zero_point, qdtype = activation_qparams(mod)
        return cls(scale, zero_point, qdtype)
