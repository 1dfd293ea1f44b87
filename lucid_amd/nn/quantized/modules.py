"""Boundary markers of a statically quantized model
(``lucid/nn/quantized/modules.py:29-424``)."""

from __future__ import annotations

import numpy as np

from ... import _C
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._qscheme import QDtype, quint8
from ..module import Module
from ._utils import host_scalar, storage_offset


class QuantStub(Module):
    """Float-model entry marker; ``prepare`` attaches its observer (a forward hook: the stub
    stays an identity), ``prepare_qat`` a ``FakeQuantize``, which the stub applies to a float
    input (``modules.py:84-95``)."""

    def forward(self, x):
        from ...quantization._fake_quantize import FakeQuantize
        app = self.__dict__.get("_modules", {}).get("activation_post_process")
        if isinstance(app, FakeQuantize) and getattr(x, "dtype", None) is T.float32:
            return app(x)
        return x


class DeQuantStub(Module):
    """Float-model exit marker."""

    def forward(self, x):
        return x


class Quantize(Module):
    """Puts a float activation on the calibrated grid (``modules.py:266-292``).
    Integer inputs (e.g. token indices) pass through unchanged."""

    def __init__(self, scale: Tensor, zero_point: Tensor, qdtype: QDtype = quint8) -> None:
        super().__init__()
        self.register_buffer("scale", scale.to("hip"))
        self.register_buffer("zero_point", zero_point.to("hip"))
        self.qdtype = qdtype
        self._zp_host = None

    def _state_loaded(self, name: str) -> None:
        if name == "zero_point":
            self._zp_host = None

    def forward(self, x: Tensor) -> Tensor:
        if not T.is_floating_point(x):
            return x
        if x.device != "hip":
            raise _C.DeviceMismatch("Quantize: input must be on the 'hip' device")
        if x.dtype != T.float32:
            raise _C.DtypeMismatch(f"Quantize expects float32, got {x.dtype}")
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.qdtype)
        if x.ndim in (4, 5):
            # an image or video batch: codes go channel-last, the layout of the conv kernels
            B, Cc = x.shape[:2]
            H, W = int(np.prod(x.shape[2:-1], dtype=np.int64)), x.shape[-1]
            codes = Tensor.empty((B, *x.shape[2:], Cc), T.int8, "hip")
            _C.call("lq_quantize_nchw_to_nhwc", x.data_ptr, codes.data_ptr, off, B, Cc, H, W,
                    self.scale.data_ptr, self.zero_point.data_ptr, self.qdtype.quant_min,
                    self.qdtype.quant_max, None)
            return Tensor.on_grid(x.shape, Grid(codes, self.scale, self.zero_point, self.qdtype,
                                                off, self._zp_host, "nhwc"))
        codes = Tensor.empty(x.shape, T.int8, "hip")
        _C.call("lq_quantize", x.data_ptr, codes.data_ptr, _C.I8, off, 1, 1, x.numel,
                self.scale.data_ptr, self.zero_point.data_ptr, 0, self.qdtype.quant_min,
                self.qdtype.quant_max, None)
        return Tensor.on_grid(x.shape, Grid(codes, self.scale, self.zero_point, self.qdtype, off,
                                            self._zp_host))

    @classmethod
    def from_float(cls, stub) -> "Quantize":
        obs = stub.activation_post_process
        scale, zero_point = obs.calculate_qparams()
        return cls(scale, zero_point, obs.qdtype)


class DeQuantize(Module):
    """Exit marker: hands back an ordinary float tensor (the float view of the
    codes is materialised here)."""

    def forward(self, x: Tensor) -> Tensor:
        if x._grid is None:
            return x
        ptr_owner = x
        ptr_owner.data_ptr  # materialise the float view
        out = Tensor(x.shape, T.float32, "hip", buf=x._buf, offset=x._offset)
        return out

    @classmethod
    def from_float(cls, stub) -> "DeQuantize":
        return cls()


class QuantWrapper(Module):
    """``QuantStub -> module -> DeQuantStub`` (``modules.py``)."""

    def __init__(self, module: Module) -> None:
        super().__init__()
        self.quant = QuantStub()
        self.module = module
        self.dequant = DeQuantStub()

    def forward(self, x):
        return self.dequant(self.module(self.quant(x)))
