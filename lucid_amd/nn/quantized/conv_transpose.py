"""Quantized ``ConvTranspose2d`` (``lucid/nn/quantized/conv_transpose.py:38-204``):
same constructor, buffers (``weight_int8`` int8 ``(in, out/groups, kh, kw)``,
``weight_scale`` / ``weight_zero_point`` f32 ``(out/groups,)`` - per channel along axis
1, shared by the groups -, ``bias``, ``scale``, ``zero_point``) and ``from_float``.

A transposed convolution is a stride-1 convolution of the zero-inserted input with the
spatially flipped kernel, input and output channels swapped inside each group, and
padding ``dilation * (k - 1) - p`` (``+ output_padding`` on the high side).  The zero
insertion is one pass over the codes (the inserted bytes are the code of real zero);
everything after it is the int8 implicit-GEMM convolution with the output requantize in
its epilogue.
"""

from __future__ import annotations

import numpy as np

from ... import _C, _ops
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._functional import quantize
from ...quantization._qscheme import QDtype, per_channel_symmetric, qint8, quint8
from ..module import Module
from ._utils import activation_qparams, host_scalar, forget_weight_zero_points, input_grid, storage_offset, weight_zero_points


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


class ConvTranspose2d(Module):
    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 output_padding=0, dilation=1, groups: int = 1, bias: bool = True) -> None:
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride, self.padding = _pair(kernel_size), _pair(stride), _pair(padding)
        self.output_padding, self.dilation, self.groups = _pair(output_padding), _pair(dilation), groups
        self.out_qdtype: QDtype = quint8
        self.weight_ch_axis = 1
        n_out = out_channels // groups
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((in_channels, n_out, *self.kernel_size), np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(n_out, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(np.zeros(n_out, np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_channels, np.float32), device="hip") if bias else None)
        self.register_buffer("scale", T.tensor(np.float32(1.0), device="hip"))
        self.register_buffer("zero_point", T.tensor(np.float32(0.0), device="hip"))
        self._w_ohwi = self._wsum = self._w_scale_full = None
        self._zp_host = None

    def _state_loaded(self, name: str) -> None:
        if name in ("weight_int8", "weight_scale"):
            self._w_ohwi = self._wsum = self._w_scale_full = None
        if name == "zero_point":
            self._zp_host = None
        if name == "weight_zero_point":
            forget_weight_zero_points(self)

    def _prepare_weight(self) -> None:
        """The equivalent convolution's kernel, ``(out, kh, kw, in/groups)``: flipped in
        space, channels swapped inside each group (one-off, on the host)."""
        w = self.weight_int8.numpy()
        cig = self.in_channels // self.groups
        blocks = [np.transpose(w[g * cig:(g + 1) * cig, :, ::-1, ::-1], (1, 2, 3, 0))
                  for g in range(self.groups)]
        self._w_ohwi = T.tensor(np.ascontiguousarray(np.concatenate(blocks, axis=0)), device="hip")
        self._wsum = _ops.rowsum_i8(self._w_ohwi)
        self._w_scale_full = T.tensor(np.tile(self.weight_scale.numpy(), self.groups), device="hip")

    def forward(self, x: Tensor) -> Tensor:
        name = type(self).__name__
        g = input_grid(x, name)
        if x.ndim != 4 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, H, W), got {x.shape}")
        if g.zp_host is None:
            raise NotImplementedError(f"{name}: the input zero point must be known on the host")
        if g.layout != "nhwc":
            raise _C.LucidError(f"{name}: 4-d activation codes must be stored NHWC")
        (kh, kw), (sh, sw), (ph, pw) = self.kernel_size, self.stride, self.padding
        (oph, opw), (dh, dw) = self.output_padding, self.dilation
        lo_h, lo_w = dh * (kh - 1) - ph, dw * (kw - 1) - pw
        if lo_h < 0 or lo_w < 0:
            raise NotImplementedError(f"{name}: padding larger than dilation * (kernel - 1) is not supported")
        if self._w_ohwi is None:
            self._prepare_weight()
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.out_qdtype)
        codes_in = g.codes
        if sh > 1 or sw > 1:
            B, H, W, Ci = codes_in.shape
            spread = Tensor.empty((B, (H - 1) * sh + 1, (W - 1) * sw + 1, Ci), T.int8, "hip")
            _C.call("lq_dilate_nhwc_i8", codes_in.data_ptr, B, H, W, Ci, sh, sw, 0, 0,
                    int(g.zp_host) + g.offset, spread.data_ptr, None)
            codes_in = spread
        codes = _ops.qconv2d_i8(
            codes_in, self._w_ohwi, a_zp=int(g.zp_host) + g.offset, a_scale=g.scale,
            w_scale=self._w_scale_full, wsum=self._wsum, bias=self.bias, stride=(1, 1),
            pad=(lo_h, lo_h + oph, lo_w, lo_w + opw), dilation=self.dilation, groups=self.groups,
            relu=False, out_mode=_ops.OUT_REQUANT_I8, out_scale=self.scale, out_zp=self.zero_point,
            out_qmin=self.out_qdtype.quant_min, out_qmax=self.out_qdtype.quant_max, out_offset=off,
            w_zp=weight_zero_points(self, self.groups))
        B, OH, OW, Co = codes.shape
        return Tensor.on_grid((B, Co, OH, OW), Grid(codes, self.scale, self.zero_point, self.out_qdtype, off,
                                                    self._zp_host, "nhwc"))

    @classmethod
    def from_float(cls, mod) -> "ConvTranspose2d":
        from ...quantization.observer import PerChannelMinMaxObserver
        if isinstance(mod.padding, str):
            raise NotImplementedError("quantized conv_transpose: string padding is not supported yet")
        q = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, mod.padding,
                mod.output_padding, mod.dilation, mod.groups, bias=mod.bias is not None)
        wobs = PerChannelMinMaxObserver(ch_axis=1, qscheme=per_channel_symmetric, qdtype=qint8)
        w = mod.weight.to("hip")
        wobs(w)
        w_scale, w_zp = wobs.calculate_qparams()
        q.register_buffer("weight_int8", quantize(w, w_scale, w_zp, qint8, ch_axis=1))
        q.register_buffer("weight_scale", w_scale.to("hip"))
        q.register_buffer("weight_zero_point", w_zp.to("hip"))
        if mod.bias is not None:
            q.register_buffer("bias", mod.bias.to("hip"))
        a_scale, a_zp, a_qdtype = activation_qparams(mod)
        q.register_buffer("scale", a_scale)
        q.register_buffer("zero_point", a_zp)
        q.out_qdtype = a_qdtype
        return q

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride}, qdtype={self.out_qdtype.name}")


class ConvTranspose1d(ConvTranspose2d):
    """Quantized ``ConvTranspose1d`` (``lucid/nn/quantized/conv_transpose.py:162-319``):
    ``weight_int8`` ``(in, out/groups, k)``; computed as the 2-d layer over a one-row image
    (codes turned to channel-last order and back)."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 output_padding=0, dilation=1, groups: int = 1, bias: bool = True) -> None:
        one = lambda v: int(v[0]) if isinstance(v, (tuple, list)) else int(v)
        super().__init__(in_channels, out_channels, (1, one(kernel_size)), (1, one(stride)), (0, one(padding)),
                         (0, one(output_padding)), (1, one(dilation)), groups, bias)
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((in_channels, out_channels // groups, one(kernel_size)), np.int8), device="hip"))

    def _prepare_weight(self) -> None:
        w3 = self.weight_int8
        try:  # the 2-d preparation on the kernel seen as (in, out/groups, 1, k)
            self._buffers["weight_int8"] = w3.reshape(w3.shape[0], w3.shape[1], 1, w3.shape[2])
            super()._prepare_weight()
        finally:
            self._buffers["weight_int8"] = w3

    def forward(self, x: Tensor) -> Tensor:
        name = type(self).__name__
        g = input_grid(x, name)
        if x.ndim != 3 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, L), got {x.shape}")
        if g.layout != "plain":
            raise _C.LucidError(f"{name}: 3-d activation codes must be stored in their own (B, C, L) order")
        B, Cc, Ln = x.shape
        nhwc = Tensor.empty((B, 1, Ln, Cc), T.int8, "hip")
        _C.call("lq_transpose_i8", g.codes.data_ptr, nhwc.data_ptr, B, Cc, Ln, Cc * Ln, Cc * Ln, None)
        x4 = Tensor.on_grid((B, Cc, 1, Ln), Grid(nhwc, g.scale, g.zero_point, g.qdtype, g.offset, g.zp_host, "nhwc"))
        y4 = super().forward(x4)
        gy = y4._grid
        _, Co, _, Lo = y4.shape
        plain = Tensor.empty((B, Co, Lo), T.int8, "hip")
        _C.call("lq_transpose_i8", gy.codes.data_ptr, plain.data_ptr, B, Lo, Co, Lo * Co, Lo * Co, None)
        return Tensor.on_grid((B, Co, Lo), Grid(plain, gy.scale, gy.zero_point, gy.qdtype, gy.offset, gy.zp_host,
                                                "plain"))

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size[1]}, "
                f"stride={self.stride[1]}, qdtype={self.out_qdtype.name}")


class ConvTranspose3d(ConvTranspose2d):
    """Quantized ``ConvTranspose3d`` (``lucid/nn/quantized/conv_transpose.py:484-640``):
    ``weight_int8`` ``(in, out/groups, kd, kh, kw)``.  The same identity as the 2-d layer - a
    stride-1 convolution of the zero-inserted input with the flipped kernel - on the
    ``(B, C, D, H, W)`` codes through the explicit-GEMM route of ``Conv3d``; the zero insertion
    happens inside the tap gather, nothing is materialised for it."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 output_padding=0, dilation=1, groups: int = 1, bias: bool = True) -> None:
        three = lambda v: (int(v),) * 3 if isinstance(v, int) else tuple(int(e) for e in v)
        super().__init__(in_channels, out_channels, (1, 1), 1, 0, 0, 1, groups, bias)
        self.kernel_size, self.stride, self.padding = three(kernel_size), three(stride), three(padding)
        self.output_padding, self.dilation = three(output_padding), three(dilation)
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((in_channels, out_channels // groups, *self.kernel_size), np.int8), device="hip"))

    def _prepare_weight(self) -> None:
        """The equivalent convolution's kernel rows ``[out, taps * in/groups]``: flipped in
        space, channels swapped inside each group (one-off, on the host)."""
        w = self.weight_int8.numpy()
        cig = self.in_channels // self.groups
        blocks = [np.transpose(w[g * cig:(g + 1) * cig, :, ::-1, ::-1, ::-1], (1, 2, 3, 4, 0))
                  for g in range(self.groups)]
        rows = np.concatenate(blocks, axis=0)
        self._w_ohwi = T.tensor(np.ascontiguousarray(rows.reshape(rows.shape[0], -1)), device="hip")
        self._wsum = _ops.rowsum_i8(self._w_ohwi)
        self._w_scale_full = T.tensor(np.tile(self.weight_scale.numpy(), self.groups), device="hip")

    def forward(self, x: Tensor) -> Tensor:
        from .conv import volumetric_gemm
        name = type(self).__name__
        g = input_grid(x, name)
        if x.ndim != 5 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, D, H, W), got {x.shape}")
        if g.zp_host is None:
            raise NotImplementedError(f"{name}: the input zero point must be known on the host")
        lo = [d * (k - 1) - p for d, k, p in zip(self.dilation, self.kernel_size, self.padding)]
        if min(lo) < 0:
            raise NotImplementedError(f"{name}: padding larger than dilation * (kernel - 1) is not supported")
        if self._w_ohwi is None:
            self._prepare_weight()
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        pads = [(l, l + op) for l, op in zip(lo, self.output_padding)]
        return volumetric_gemm(name, x, g, self._w_ohwi, self._wsum, self._w_scale_full, self.bias, self.kernel_size,
                               (1, 1, 1), pads, self.dilation, self.stride, self.groups, False, self.scale,
                               self.zero_point, self.out_qdtype, self._zp_host,
                               w_zp=weight_zero_points(self, self.groups))
