"""Quantized ``Linear`` for static PTQ, on the hip int8 GEMM.

Mirrors ``lucid/nn/quantized/linear.py:171-243``: same constructor, buffer
names and dtypes (``weight_int8`` int8 (N,K); ``weight_scale`` /
``weight_zero_point`` f32 (N,); ``bias`` f32 (N,) or None; ``scale`` /
``zero_point`` f32 0-d), attributes ``weight_ch_axis`` and ``out_qdtype``,
``from_float`` and the ``_activation`` hook.  Lucid's forward dequantizes the
weight, runs a float GEMM and fake-quantizes the result; here the same
function is one int8 x int8 -> int32 MFMA GEMM whose epilogue applies the
zero-point correction, scales, bias, optional ReLU and the output requantize.
"""

from __future__ import annotations

import numpy as np

from ... import _C, _ops
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._qscheme import QDtype, quint8
from ..module import Module
from ._utils import (activation_qparams, host_scalar, input_grid, quantize_weight,
                     forget_weight_zero_points, storage_offset, weight_zero_points, zp_args)


class Linear(Module):
    _fused_relu = False

    def __init__(self, in_features: int, out_features: int, bias: bool = True) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight_ch_axis = 0
        self.out_qdtype: QDtype = quint8
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((out_features, in_features), np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(out_features, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(
            np.zeros(out_features, np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_features, np.float32), device="hip")
                             if bias else None)
        self.register_buffer("scale", T.tensor(np.float32(1.0), device="hip"))
        self.register_buffer("zero_point", T.tensor(np.float32(0.0), device="hip"))
        self._wsum = None     # int32 row sums of weight_int8 (derived, not in state_dict)
        self._zp_host = None  # host copy of zero_point

    def _state_loaded(self, name: str) -> None:
        if name == "weight_int8":
            self._wsum = None
        if name == "zero_point":
            self._zp_host = None
        if name == "weight_zero_point":
            forget_weight_zero_points(self)

    def _activation(self, y: Tensor) -> Tensor:
        """Post-linear activation hook (identity; ReLU in the fused variant).
        Kept for API parity; the hip forward fuses the ReLU into the GEMM."""
        return y

    def _forward_float(self, x: Tensor) -> Tensor:
        """Input is a float tensor on no grid (e.g. after global average
        pooling): Lucid's own formulation - dequantized weight, float GEMM,
        fake-quantized output - in one small kernel."""
        K, N = self.in_features, self.out_features
        M = x.numel // K
        y = Tensor.empty((M, N), T.float32, "hip")
        _C.call("lq_qlinear_w8a32", x.data_ptr, self.weight_int8.data_ptr,
                self.weight_scale.data_ptr, self.weight_zero_point.data_ptr,
                self.bias.data_ptr if self.bias is not None else None, M, N, K,
                int(self._fused_relu), 1, self.scale.data_ptr, self.zero_point.data_ptr,
                self.out_qdtype.quant_min, self.out_qdtype.quant_max, y.data_ptr, None)
        return y.reshape(*x.shape[:-1], N)

    def forward(self, x: Tensor) -> Tensor:
        K, N = self.in_features, self.out_features
        if not isinstance(x, Tensor) or x.device != "hip":
            raise _C.DeviceMismatch(f"{type(self).__name__}: input must be on the 'hip' device")
        if x.shape[-1] != K:
            raise _C.ShapeMismatch(f"expected last dim {K}, got {x.shape}")
        if x._grid is None or x._grid.layout != "plain":
            if x.dtype != T.float32:
                raise _C.DtypeMismatch(f"{type(self).__name__} expects float32, got {x.dtype}")
            return self._forward_float(x)
        g = x._grid
        M = x.numel // K
        if self._wsum is None:
            self._wsum = _ops.rowsum_i8(self.weight_int8)
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        a_zp, a_zp_dev = zp_args(g)
        off = storage_offset(self.out_qdtype)
        codes = _ops.qlinear_i8(
            g.codes.reshape(M, K), self.weight_int8, a_zp=a_zp, a_zp_dev=a_zp_dev,
            a_scale=g.scale, w_scale=self.weight_scale, wsum=self._wsum, bias=self.bias,
            relu=self._fused_relu, out_mode=_ops.OUT_REQUANT_I8, out_scale=self.scale,
            out_zp=self.zero_point, out_qmin=self.out_qdtype.quant_min,
            out_qmax=self.out_qdtype.quant_max, out_offset=off, w_zp=weight_zero_points(self))
        shape = x.shape[:-1] + (N,)
        return Tensor.on_grid(shape, Grid(codes.reshape(shape), self.scale, self.zero_point,
                                          self.out_qdtype, off, self._zp_host))

    @classmethod
    def from_float(cls, mod) -> "Linear":
        """Quantize a calibrated float ``Linear`` (``linear.py:217-236``)."""
        has_bias = mod.bias is not None
        qmod = cls(mod.in_features, mod.out_features, bias=has_bias)
        codes, w_scale, w_zp, ch_axis = quantize_weight(mod)
        qmod.register_buffer("weight_int8", codes)
        qmod.register_buffer("weight_scale", w_scale)
        qmod.register_buffer("weight_zero_point", w_zp)
        qmod.weight_ch_axis = ch_axis
        if has_bias:
            qmod.register_buffer("bias", mod.bias.to("hip"))  # bias stays float
        a_scale, a_zp, a_qdtype = activation_qparams(mod)
        qmod.register_buffer("scale", a_scale)
        qmod.register_buffer("zero_point", a_zp)
        qmod.out_qdtype = a_qdtype
        return qmod

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"qdtype={self.out_qdtype.name}")
