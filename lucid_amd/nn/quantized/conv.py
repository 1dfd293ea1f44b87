"""Quantized ``Conv2d`` for static PTQ, on the hip implicit-GEMM int8 kernel.

Mirrors ``lucid/nn/quantized/conv.py:75-229,388-542``: same constructor,
buffers (``weight_int8`` int8 ``(Cout, Cin/groups, KH, KW)`` - Lucid's OIHW
order is kept as the state-dict contract -, ``weight_scale`` /
``weight_zero_point`` f32 ``(Cout,)``, ``bias``, ``scale``, ``zero_point``),
attributes ``padding_str`` / ``padding_mode`` / ``weight_ch_axis`` /
``out_qdtype``, ``from_float`` and the ``_activation`` hook.  The forward is
one launch: activation codes (NHWC) x repacked weight codes through the MFMA
GEMM with zero-point correction, scales, bias, optional ReLU and the output
requantize in the epilogue.
"""

from __future__ import annotations

import ctypes as C

import numpy as np

from ... import _C, _ops
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._qscheme import QDtype, quint8
from ..module import Module
from ._utils import (activation_qparams, float_input_conv, host_scalar, input_grid, is_plain_float, plain_volume_grid, quantize_weight,
                     forget_weight_zero_points, storage_offset, weight_zero_points)


_PAD_MODES = {"zeros": 0, "reflect": 1, "replicate": 2, "circular": 3}


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def _same_pad_pair(in_size: int, kernel: int, stride: int, dilation: int) -> tuple[int, int]:
    """``padding="same"`` amounts (``lucid/nn/modules/conv.py:44-55``): the odd
    unit goes to the high side."""
    out_size = (in_size + stride - 1) // stride
    pad_total = max(0, (out_size - 1) * stride + (kernel - 1) * dilation + 1 - in_size)
    return pad_total // 2, pad_total - pad_total // 2


class Conv2d(Module):
    _fused_relu = False

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 dilation=1, groups: int = 1, bias: bool = True) -> None:
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = _pair(kernel_size), _pair(stride)
        self.padding_str = padding if isinstance(padding, str) else None
        self.padding = (0, 0) if isinstance(padding, str) else _pair(padding)
        self.dilation, self.groups = _pair(dilation), groups
        self.padding_mode = "zeros"
        self.weight_ch_axis = 0
        self.out_qdtype: QDtype = quint8
        wshape = (out_channels, in_channels // groups, *self.kernel_size)
        self.register_buffer("weight_int8", T.tensor(np.zeros(wshape, np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(out_channels, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(
            np.zeros(out_channels, np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_channels, np.float32), device="hip")
                             if bias else None)
        self.register_buffer("scale", T.tensor(np.float32(1.0), device="hip"))
        self.register_buffer("zero_point", T.tensor(np.float32(0.0), device="hip"))
        self._w_ohwi = None   # weight codes repacked to (Cout, KH, KW, Cin/groups)
        self._wsum = None
        self._zp_host = None

    def _state_loaded(self, name: str) -> None:
        if name == "weight_int8":
            self._w_ohwi = self._wsum = None
            self.__dict__.pop("_w_packed4", None)
        if name == "zero_point":
            self._zp_host = None
        if name == "weight_zero_point":
            forget_weight_zero_points(self)
        if name in ("weight_int8", "weight_scale", "weight_zero_point"):
            self.__dict__.pop("_w_float", None)      # the float-input form's dequantized weight
        if name in ("scale", "zero_point"):
            self.__dict__.pop("_out_quantize", None)

    def _resolve_pad(self, x: Tensor) -> tuple[int, int, int, int]:
        """(h_lo, h_hi, w_lo, w_hi), as ``conv.py:119-141``."""
        if self.padding_str == "valid":
            return 0, 0, 0, 0
        if self.padding_str == "same":
            h = _same_pad_pair(x.shape[2], self.kernel_size[0], self.stride[0], self.dilation[0])
            w = _same_pad_pair(x.shape[3], self.kernel_size[1], self.stride[1], self.dilation[1])
            return h[0], h[1], w[0], w[1]
        return self.padding[0], self.padding[0], self.padding[1], self.padding[1]

    def _activation(self, y: Tensor) -> Tensor:
        """Post-conv activation hook (identity; ReLU in the fused variant)."""
        return y

    def _prepare_weight(self) -> None:
        O, I, KH, KW = self.weight_int8.shape
        w = Tensor.empty((O, KH, KW, I), T.int8, "hip")
        _C.call("lq_repack_oihw_to_ohwi_i8", self.weight_int8.data_ptr, w.data_ptr, O, I, KH, KW, None)
        self._w_ohwi = w
        self._wsum = _ops.rowsum_i8(w)

    def _forward_quantizing(self, x: Tensor, quantize) -> Tensor | None:
        """``self(quantize(x))`` for a float image of at most four channels without the NHWC code
        tensor in between: the image is quantized straight into the packed, pre-padded form the
        few-channel kernel route gathers from (one pass instead of quantize + pack, and the
        filter is packed once).  None where that route does not take the layer."""
        KH, KW = self.kernel_size
        if type(self).forward is not Conv2d.forward or not is_plain_float(x) \
                or x.ndim != 4 or x.shape[1] != self.in_channels or x.dtype != T.float32 or x.device != "hip" \
                or self.in_channels > 4 or self.groups != 1 or self.dilation[1] != 1 \
                or self.padding_mode != "zeros" or KH * ((KW + 3) // 4) * 16 > 131071 \
                or weight_zero_points(self) is not None or x.numel == 0:
            return None
        if self._w_ohwi is None:
            self._prepare_weight()
        if self.__dict__.get("_w_packed4") is None:
            self._w_packed4 = _ops.pack4_filter_i8(self._w_ohwi)
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        if quantize._zp_host is None:
            quantize._zp_host = int(host_scalar(quantize.zero_point))
        qd, qoff = quantize.qdtype, storage_offset(quantize.qdtype)
        pad = self._resolve_pad(x)
        B, Cc, H, W = x.shape
        if _ops.conv_out_size(H, KH, self.stride[0], pad[0], pad[1], self.dilation[0]) <= 0 or \
                _ops.conv_out_size(W, KW, self.stride[1], pad[2], pad[3], 1) <= 0:
            return None
        Hp, Wp, _ = _ops.packed4_geometry(H, W, Cc, KW, self.stride[1], pad)
        a_zp = quantize._zp_host + qoff
        image = _ops.quantize_nchw_to_packed4(x, quantize.scale, quantize.zero_point, qd.quant_min, qd.quant_max,
                                              qoff, a_zp, pad, Hp, Wp)
        off = storage_offset(self.out_qdtype)
        codes = _ops.qconv2d_i8(
            image, self._w_packed4, a_zp=a_zp, a_scale=quantize.scale, w_scale=self.weight_scale, wsum=self._wsum,
            bias=self.bias, stride=self.stride, pad=pad, dilation=self.dilation, relu=self._fused_relu,
            out_mode=_ops.OUT_REQUANT_I8, out_scale=self.scale, out_zp=self.zero_point,
            out_qmin=self.out_qdtype.quant_min, out_qmax=self.out_qdtype.quant_max, out_offset=off,
            path=_ops.CONV_PREPACKED4, logical=(H, W, Cc, KW))
        _, OH, OW, Co = codes.shape
        return Tensor.on_grid((B, Co, OH, OW), Grid(codes, self.scale, self.zero_point,
                                                    self.out_qdtype, off, self._zp_host, "nhwc"))

    def forward(self, x: Tensor, join=None, quantize=None) -> Tensor:
        """``join = (other, qfunctional, relu)`` fuses ``qfunctional.add[_relu](self(x), other)``
        into this layer's epilogue: the result is on the functional's grid, bit for bit what
        the two separate modules give, and the layer's own output is never stored.
        ``quantize`` (a ``Quantize`` module) stands for ``self(quantize(x))`` on a float ``x``:
        the same codes, and for a first layer of at most four channels one pass less."""
        if quantize is not None:
            if join is None:
                fused = self._forward_quantizing(x, quantize)
                if fused is not None:
                    return fused
            x = quantize(x)
        name = type(self).__name__
        if is_plain_float(x) and join is None:
            # no grid on the input: Lucid's float formulation (conv.py:168-184)
            if x.ndim != 4 or x.shape[1] != self.in_channels:
                raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, H, W), got {x.shape}")
            p = self._resolve_pad(x)
            return float_input_conv(self, x, 2, ((p[0], p[1]), (p[2], p[3])), self._fused_relu)
        g = input_grid(x, name)
        if x.ndim != 4 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, H, W), got {x.shape}")
        if self.padding_mode not in _PAD_MODES:
            raise ValueError(f"{name}: unknown padding_mode {self.padding_mode!r}")
        if g.zp_host is None:
            raise NotImplementedError(
                f"{name}: the input zero point is only known on the device; convolution needs it "
                "on the host for the padding code (static quantization provides it)")
        if g.layout != "nhwc":
            raise _C.LucidError(f"{name}: 4-d activation codes must be stored NHWC")
        if self._w_ohwi is None:
            self._prepare_weight()
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        off = storage_offset(self.out_qdtype)
        in_codes, pad = g.codes, self._resolve_pad(x)
        if self.padding_mode != "zeros" and any(pad):
            # pre-pad the codes, then convolve with padding 0 (nn/modules/conv.py:104-123)
            B, H, W, Ci = in_codes.shape
            padded = Tensor.empty((B, H + pad[0] + pad[1], W + pad[2] + pad[3], Ci), T.int8, "hip")
            _C.call("lq_pad_nhwc_i8", in_codes.data_ptr, padded.data_ptr, B, H, W, Ci, pad[0], pad[1], pad[2],
                    pad[3], _PAD_MODES[self.padding_mode], None)
            in_codes, pad = padded, (0, 0, 0, 0)
        jarg = out_grid = None
        if join is not None:
            other, fn, relu = join
            go = input_grid(other, name)
            if go.layout != "nhwc":
                raise _C.LucidError(f"{name}: the joined operand's codes must be stored NHWC")
            if fn._zp_host is None:
                fn._zp_host = int(host_scalar(fn.zero_point))
            foff = storage_offset(fn.qdtype)
            jarg = dict(q=go.codes, offset=go.offset, scale=go.scale, zp=go.zero_point, relu=relu,
                        out_scale=fn.scale, out_zp=fn.zero_point, out_qmin=fn.qdtype.quant_min,
                        out_qmax=fn.qdtype.quant_max, out_offset=foff)
            out_grid = (fn.scale, fn.zero_point, fn.qdtype, foff, fn._zp_host)
        codes = _ops.qconv2d_i8(
            in_codes, self._w_ohwi, a_zp=int(g.zp_host) + g.offset, a_scale=g.scale,
            w_scale=self.weight_scale, wsum=self._wsum, bias=self.bias, stride=self.stride,
            pad=pad, dilation=self.dilation, groups=self.groups,
            relu=self._fused_relu, out_mode=_ops.OUT_REQUANT_I8, out_scale=self.scale,
            out_zp=self.zero_point, out_qmin=self.out_qdtype.quant_min,
            out_qmax=self.out_qdtype.quant_max, out_offset=off, join=jarg, w_zp=weight_zero_points(self))
        B, OH, OW, Co = codes.shape
        if out_grid is not None:
            return Tensor.on_grid((B, Co, OH, OW), Grid(codes, *out_grid, "nhwc"))
        return Tensor.on_grid((B, Co, OH, OW), Grid(codes, self.scale, self.zero_point,
                                                    self.out_qdtype, off, self._zp_host, "nhwc"))

    @classmethod
    def from_float(cls, mod) -> "Conv2d":
        """Quantize a calibrated float ``Conv2d`` (``conv.py:186-222``)."""
        qmod = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, mod.padding,
                   mod.dilation, mod.groups, bias=mod.bias is not None)
        codes, w_scale, w_zp, ch_axis = quantize_weight(mod)
        qmod.register_buffer("weight_int8", codes)
        qmod.register_buffer("weight_scale", w_scale)
        qmod.register_buffer("weight_zero_point", w_zp)
        qmod.weight_ch_axis = ch_axis
        qmod.padding_str = getattr(mod, "_padding_str", None)
        qmod.padding_mode = getattr(mod, "padding_mode", "zeros")
        if mod.bias is not None:
            qmod.register_buffer("bias", mod.bias.to("hip"))
        a_scale, a_zp, a_qdtype = activation_qparams(mod)
        qmod.register_buffer("scale", a_scale)
        qmod.register_buffer("zero_point", a_zp)
        qmod.out_qdtype = a_qdtype
        return qmod

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride}, qdtype={self.out_qdtype.name}")


class Conv1d(Conv2d):
    """Quantized ``Conv1d`` (``lucid/nn/quantized/conv.py:232-385``): the same buffers with a
    three-dimensional kernel ``weight_int8`` ``(Cout, Cin/groups, K)``.  A 1-d convolution over
    ``(B, C, L)`` is the 2-d one over ``(B, C, 1, L)``: the input codes are turned to
    channel-last order, the implicit-GEMM kernel runs with a one-row image, and the result is
    turned back to ``(B, Cout, L_out)`` codes."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 dilation=1, groups: int = 1, bias: bool = True) -> None:
        one = lambda v: int(v[0]) if isinstance(v, (tuple, list)) else int(v)
        super().__init__(in_channels, out_channels, (1, one(kernel_size)), (1, one(stride)),
                         padding if isinstance(padding, str) else (0, one(padding)), (1, one(dilation)), groups, bias)
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((out_channels, in_channels // groups, one(kernel_size)), np.int8), device="hip"))

    def _prepare_weight(self) -> None:
        O, I, K = self.weight_int8.shape
        w = Tensor.empty((O, 1, K, I), T.int8, "hip")
        _C.call("lq_repack_oihw_to_ohwi_i8", self.weight_int8.data_ptr, w.data_ptr, O, I, 1, K, None)
        self._w_ohwi = w
        self._wsum = _ops.rowsum_i8(w)

    def forward(self, x: Tensor) -> Tensor:
        name = type(self).__name__
        if is_plain_float(x):
            if x.ndim != 3 or x.shape[1] != self.in_channels:
                raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, L), got {x.shape}")
            p = self._resolve_pad(x.reshape(x.shape[0], x.shape[1], 1, x.shape[2]))
            return float_input_conv(self, x, 1, ((p[2], p[3]),), self._fused_relu)
        g = input_grid(x, name)
        if x.ndim != 3 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, L), got {x.shape}")
        if g.layout != "plain":
            raise _C.LucidError(f"{name}: 3-d activation codes must be stored in their own (B, C, L) order")
        B, Cc, Ln = x.shape
        # (B, C, L) -> (B, 1, L, C): a batched byte transpose
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

    @classmethod
    def from_float(cls, mod) -> "Conv1d":
        """Quantize a calibrated float ``Conv1d`` (``conv.py:186-222``)."""
        qmod = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, mod.padding,
                   mod.dilation, mod.groups, bias=mod.bias is not None)
        codes, w_scale, w_zp, ch_axis = quantize_weight(mod)
        qmod.register_buffer("weight_int8", codes)
        qmod.register_buffer("weight_scale", w_scale)
        qmod.register_buffer("weight_zero_point", w_zp)
        qmod.weight_ch_axis = ch_axis
        qmod.padding_str = getattr(mod, "_padding_str", None)
        qmod.padding_mode = getattr(mod, "padding_mode", "zeros")
        if mod.bias is not None:
            qmod.register_buffer("bias", mod.bias.to("hip"))
        a_scale, a_zp, a_qdtype = activation_qparams(mod)
        qmod.register_buffer("scale", a_scale)
        qmod.register_buffer("zero_point", a_zp)
        qmod.out_qdtype = a_qdtype
        return qmod

    def extra_repr(self) -> str:
        return (f"{self.in_channels}, {self.out_channels}, kernel_size={self.kernel_size[1]}, "
                f"stride={self.stride[1]}, qdtype={self.out_qdtype.name}")


def _triple(v):
    return (int(v),) * 3 if isinstance(v, int) else tuple(int(e) for e in v)


def volumetric_gemm(name, x: Tensor, g, w_rows: Tensor, wsum: Tensor, w_scale: Tensor, bias, kernel, stride,
                    pads, dilation, insert, groups: int, relu: bool, scale: Tensor, zero_point: Tensor,
                    qdtype: QDtype, zp_host: int, w_zp: Tensor | None = None) -> Tensor:
    """A 3-d convolution on codes.  With ``C/groups`` a multiple of 16 and no insertion: one
    fused launch whose loader gathers the taps (``lq_qconv3d_i8``), the result kept channels-last
    (layout "nhwc").  Otherwise as an explicit
    GEMM, group by group: gather the taps of
    ``x``'s ``(B, C, D, H, W)`` codes (``insert`` > 1: as if zero-point codes stood between
    neighbouring samples), multiply with the group's kernel rows ``[Cout/groups, taps * C/groups]``
    through the fused int8 GEMM, write the result channels-first.  The codes are turned
    channels-last first, so that the gather moves contiguous runs.  ``pads`` = ((lo, hi),) * 3."""
    B, Cc, D, H, W = x.shape
    spread = [(n - 1) * i + 1 for n, i in zip((D, H, W), insert)]
    outs = [(n + lo + hi - d * (k - 1) - 1) // s + 1
            for n, (lo, hi), k, s, d in zip(spread, pads, kernel, stride, dilation)]
    if min(outs) < 1:
        raise _C.ShapeMismatch(f"{name}: kernel {tuple(kernel)} does not fit input {x.shape}")
    L = outs[0] * outs[1] * outs[2]
    Co = w_rows.shape[0]
    Cg, Og = Cc // groups, Co // groups
    a_zp = int(g.zp_host) + g.offset
    off = storage_offset(qdtype)
    i3 = lambda v: (C.c_int * 3)(*[int(e) for e in v])
    vol = D * H * W
    if g.layout == "nhwc":
        last = g.codes                                        # already (B, D, H, W, C)
    else:
        last = Tensor.empty((B, D, H, W, Cc), T.int8, "hip")  # channels-last copy of the input codes
        _C.call("lq_transpose_i8", g.codes.data_ptr, last.data_ptr, B, Cc, vol, Cc * vol, Cc * vol, None)
    if Cg % 16 == 0 and tuple(insert) == (1, 1, 1):
        # the taps are gathered by the GEMM's loader (no patch matrix), all groups in one launch
        w5 = w_rows.reshape((Co, *[int(k) for k in kernel], Cg))
        y = _ops.qconv3d_i8(last, w5, a_zp=a_zp, a_scale=g.scale, w_scale=w_scale, wsum=wsum, bias=bias,
                            stride=stride, pad=pads, dilation=dilation, groups=groups, relu=relu,
                            out_mode=_ops.OUT_REQUANT_I8, out_scale=scale, out_zp=zero_point,
                            out_qmin=qdtype.quant_min, out_qmax=qdtype.quant_max, out_offset=off, w_zp=w_zp)
        # the result stays channels-last: the next volumetric layer reads it as it is
        return Tensor.on_grid((B, Co, *outs), Grid(y, scale, zero_point, qdtype, off, zp_host, "nhwc"))
    codes = Tensor.empty((B, Co, *outs), T.int8, "hip")
    cols = Tensor.empty((B * L, Cg * kernel[0] * kernel[1] * kernel[2]), T.int8, "hip")
    for grp in range(groups):
        _C.call("lq_im2col_ndhwc_i8", last.data_ptr, cols.data_ptr, B, D, H, W, Cc, grp * Cg, Cg, i3(kernel),
                i3(stride), i3([p[0] for p in pads]), i3(dilation), i3(insert), i3(outs), a_zp, None)
        part = lambda t: t.row_range(grp * Og, (grp + 1) * Og)
        y = _ops.qlinear_i8(cols, part(w_rows), a_zp=a_zp, a_scale=g.scale, w_scale=part(w_scale), wsum=part(wsum),
                            bias=None if bias is None else part(bias), relu=relu, out_mode=_ops.OUT_REQUANT_I8,
                            out_scale=scale, out_zp=zero_point, out_qmin=qdtype.quant_min,
                            out_qmax=qdtype.quant_max, out_offset=off, w_zp=None if w_zp is None else part(w_zp))
        # each batch's [L, Og] block -> its (Og, L) channel slice of the (B, Co, L) output
        _C.call("lq_transpose_i8", y.data_ptr, codes.data_ptr + grp * Og * L, B, L, Og, L * Og, Co * L, None)
    return Tensor.on_grid((B, Co, *outs), Grid(codes, scale, zero_point, qdtype, off, zp_host, "plain"))


class Conv3d(Conv2d):
    """Quantized ``Conv3d`` (``lucid/nn/quantized/conv.py:545-700``): the same buffers with a
    five-dimensional kernel ``weight_int8`` ``(Cout, Cin/groups, KD, KH, KW)``.  The forward is
    an explicit GEMM on codes: the taps of each group are gathered from the ``(B, C, D, H, W)``
    codes into a matrix (padding taps hold the input zero point's code), multiplied with the
    group's kernel rows by the int8 GEMM with the usual fused epilogue (zero-point correction,
    scales, bias, optional ReLU, requantize) and written back channels-first.  Zero padding
    only (numbers, ``"same"`` or ``"valid"``)."""

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 dilation=1, groups: int = 1, bias: bool = True) -> None:
        super().__init__(in_channels, out_channels, (1, 1), (1, 1), 0, (1, 1), groups, bias)
        self.kernel_size, self.stride = _triple(kernel_size), _triple(stride)
        self.padding_str = padding if isinstance(padding, str) else None
        self.padding = (0, 0, 0) if isinstance(padding, str) else _triple(padding)
        self.dilation = _triple(dilation)
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((out_channels, in_channels // groups, *self.kernel_size), np.int8), device="hip"))

    def _prepare_weight(self) -> None:
        O, I, KD, KH, KW = self.weight_int8.shape
        w = Tensor.empty((O, KD * KH * KW * I), T.int8, "hip")
        _C.call("lq_repack_oihw_to_ohwi_i8", self.weight_int8.data_ptr, w.data_ptr, O, I, 1, KD * KH * KW, None)
        self._w_ohwi = w
        self._wsum = _ops.rowsum_i8(w)

    def _resolve_pad3(self, sizes) -> list[tuple[int, int]]:
        if self.padding_str == "valid":
            return [(0, 0)] * 3
        if self.padding_str == "same":
            return [_same_pad_pair(n, k, s, d)
                    for n, k, s, d in zip(sizes, self.kernel_size, self.stride, self.dilation)]
        return [(p, p) for p in self.padding]

    def forward(self, x: Tensor) -> Tensor:
        name = type(self).__name__
        if is_plain_float(x):
            if x.ndim != 5 or x.shape[1] != self.in_channels:
                raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, D, H, W), got {x.shape}")
            return float_input_conv(self, x, 3, self._resolve_pad3(x.shape[2:]), self._fused_relu)
        g = input_grid(x, name)
        if x.ndim != 5 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"{name}: expected (B, {self.in_channels}, D, H, W), got {x.shape}")
        if self.padding_mode not in _PAD_MODES:
            raise ValueError(f"{name}: unknown padding_mode {self.padding_mode!r}")
        if g.zp_host is None:
            raise NotImplementedError(
                f"{name}: the input zero point is only known on the device; convolution needs it "
                "on the host for the padding code (static quantization provides it)")
        if self._w_ohwi is None:
            self._prepare_weight()
        if self._zp_host is None:
            self._zp_host = int(host_scalar(self.zero_point))
        pads = self._resolve_pad3(x.shape[2:])
        if self.padding_mode != "zeros" and any(lo or hi for lo, hi in pads):
            g = plain_volume_grid(x, g)
            # pre-pad the codes, then convolve with padding 0 (nn/modules/conv.py:104-123).  F.pad's
            # reflect / replicate / circular act on one axis at a time, so the volume is padded in
            # two passes of the 2-d kernel: (H, W) with every (b, c, d) plane as an image of one
            # channel, then D with every (b, c) volume as a one-column image whose "channels" are
            # the padded planes.
            B, Cc, D, H, W = x.shape
            (d_lo, d_hi), (h_lo, h_hi), (w_lo, w_hi) = pads
            Hp, Wp = H + h_lo + h_hi, W + w_lo + w_hi
            mode = _PAD_MODES[self.padding_mode]
            hw = Tensor.empty((B, Cc, D, Hp, Wp), T.int8, "hip")
            _C.call("lq_pad_nhwc_i8", g.codes.data_ptr, hw.data_ptr, B * Cc * D, H, W, 1, h_lo, h_hi, w_lo, w_hi, mode,
                    None)
            full = Tensor.empty((B, Cc, D + d_lo + d_hi, Hp, Wp), T.int8, "hip")
            _C.call("lq_pad_nhwc_i8", hw.data_ptr, full.data_ptr, B * Cc, D, 1, Hp * Wp, d_lo, d_hi, 0, 0, mode, None)
            g = Grid(full, g.scale, g.zero_point, g.qdtype, g.offset, g.zp_host, "plain")
            x = Tensor.on_grid(full.shape, g)
            pads = [(0, 0)] * 3
        return volumetric_gemm(name, x, g, self._w_ohwi, self._wsum, self.weight_scale, self.bias, self.kernel_size,
                               self.stride, pads, self.dilation, (1, 1, 1), self.groups, self._fused_relu,
                               self.scale, self.zero_point, self.out_qdtype, self._zp_host,
                               w_zp=weight_zero_points(self))

    @classmethod
    def from_float(cls, mod) -> "Conv3d":
        """Quantize a calibrated float ``Conv3d`` (``conv.py:186-222``)."""
        qmod = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, mod.padding,
                   mod.dilation, mod.groups, bias=mod.bias is not None)
        codes, w_scale, w_zp, ch_axis = quantize_weight(mod)
        qmod.register_buffer("weight_int8", codes)
        qmod.register_buffer("weight_scale", w_scale)
        qmod.register_buffer("weight_zero_point", w_zp)
        qmod.weight_ch_axis = ch_axis
        qmod.padding_str = getattr(mod, "_padding_str", None)
        qmod.padding_mode = getattr(mod, "padding_mode", "zeros")
        if mod.bias is not None:
            qmod.register_buffer("bias", mod.bias.to("hip"))
        a_scale, a_zp, a_qdtype = activation_qparams(mod)
        qmod.register_buffer("scale", a_scale)
        qmod.register_buffer("zero_point", a_zp)
        qmod.out_qdtype = a_qdtype
        return qmod
