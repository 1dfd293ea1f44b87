"""Helpers shared by the quantized modules (``lucid/nn/quantized/_utils.py``)."""

from __future__ import annotations

import warnings

import numpy as np

from ... import _C, _ops
from ... import _tensor as T
from ..._tensor import Grid, Tensor
from ...quantization._functional import quantize
from ...quantization._qscheme import QDtype


def storage_offset(qdtype: QDtype) -> int:
    """What is added to a code so that it fits a signed int8 MFMA operand."""
    if qdtype.bits > 8:
        raise NotImplementedError(f"{qdtype!r} activations do not fit the int8 kernels")
    return 0 if qdtype.signed else -(1 << (qdtype.bits - 1))


def quantize_weight(mod) -> tuple[Tensor, Tensor, Tensor, int]:
    """``(codes, scale, zero_point, ch_axis)`` of a float module's weight
    (``_utils.py:27-55``): run the qconfig's weight observer over the static
    weight, then ``quantize`` along its channel axis."""
    weight = mod.weight.to("hip")
    wobs = getattr(mod, "weight_fake_quant", None)  # a QAT layer: its FakeQuantize, refreshed
    if wobs is None:
        wobs = mod.qconfig.weight()
    wobs(weight)
    scale, zero_point = wobs.calculate_qparams()
    qdtype, ch_axis = wobs.qdtype, wobs.ch_axis
    axis = ch_axis if ch_axis is not None else 0
    if qdtype.storage != "int8":
        raise NotImplementedError(f"weights must quantize to int8 storage, got {qdtype!r}")
    codes = quantize(weight, scale, zero_point, qdtype, ch_axis=ch_axis)
    if ch_axis is None:  # per-tensor weight qparams: broadcast to one entry per output row
        n = weight.shape[0]
        scale = T.tensor(np.full(n, scale.item(), np.float32), device="hip")
        zero_point = T.tensor(np.full(n, zero_point.item(), np.float32), device="hip")
    return codes, scale, zero_point, axis


def activation_qparams(mod) -> tuple[Tensor, Tensor, QDtype]:
    """Output ``(scale, zero_point, qdtype)`` from a module's activation
    observer (``_utils.py:58-79``), with Lucid's uncalibrated-observer warning."""
    obs = mod.activation_post_process
    min_val = getattr(obs, "min_val", None)
    if min_val is not None and bool(np.isinf(min_val.numpy()).any()):
        warnings.warn(
            f"Quantizing {type(mod).__name__} whose activation observer never saw "
            "data — run calibration through the prepared model before convert(), "
            "or the quantized output collapses to a near-zero grid.",
            stacklevel=3,
        )
    scale, zero_point = obs.calculate_qparams()
    return scale.to("hip"), zero_point.to("hip"), obs.qdtype


_UNSET = object()


def weight_zero_points(mod, tile: int = 1) -> Tensor | None:
    """The zero points of a module's weight rows as the int32 device vector the int8
    kernels take, or ``None`` when every one is zero (symmetric weights, Lucid's default:
    the kernels then skip the activation sums).  ``tile`` repeats the vector (the
    per-group copies of a transposed convolution's channels).  Cached on the module until
    ``weight_zero_point`` is loaded again."""
    cached = mod.__dict__.get("_wzp", _UNSET)
    if cached is not _UNSET:
        return cached
    z = mod.weight_zero_point.numpy().reshape(-1).astype(np.float64)
    if not np.any(z != 0):
        wzp = None
    else:
        zi = np.rint(z)
        if np.any(zi != z) or zi.min() < -128 or zi.max() > 127:
            raise ValueError(f"{type(mod).__name__}: weight zero points must be int8 codes, got "
                             f"values in [{z.min()}, {z.max()}]")
        wzp = T.tensor(np.tile(zi.astype(np.int32), tile), device="hip")
    mod.__dict__["_wzp"] = wzp
    return wzp


def forget_weight_zero_points(mod) -> None:
    mod.__dict__.pop("_wzp", None)


def is_plain_float(x) -> bool:
    """A float32 device tensor that carries no quantization grid: the input for which a quantized
    layer takes Lucid's float formulation."""
    return isinstance(x, Tensor) and x.device == "hip" and x._grid is None and x.dtype == T.float32


def float_input_conv(mod, x: Tensor, nd: int, pads, relu: bool) -> Tensor:
    """A quantized convolution on a plain float input, as Lucid writes it
    (``lucid/nn/quantized/conv.py:168-184``): dequantize the weight, convolve in float32 with the
    bias, optionally ReLU, fake-quantize the result to the layer's output grid - returned as a
    tensor on that grid (its float view is the fake-quantized value).  ``pads`` = per spatial
    axis ``(lo, hi)``; a padding mode other than zeros, or uneven amounts, pre-pad the input
    (``lucid/nn/modules/conv.py:104-123``).  The float32 convolution sums in another order than
    Lucid's GEMM, so codes can differ by one step where a value sits on a rounding tie."""
    from ...quantization._functional import dequantize
    from .. import functional as F
    from .modules import Quantize

    name = type(mod).__name__
    w = mod.__dict__.get("_w_float")
    if w is None:
        w = dequantize(mod.weight_int8, mod.weight_scale, mod.weight_zero_point, ch_axis=0)
        mod.__dict__["_w_float"] = w
    mode = {"zeros": 0, "reflect": 1, "replicate": 2, "circular": 3}[mod.padding_mode]
    sym = all(lo == hi for lo, hi in pads)
    conv_pad = tuple(lo for lo, _ in pads)
    if any(lo or hi for lo, hi in pads) and (mode != 0 or not sym):
        if nd == 3 and (pads[0][0] or pads[0][1]):
            raise NotImplementedError(f"{name}: a float input with padding_mode={mod.padding_mode!r} or uneven "
                                      "padding along the depth axis; quantize the input first (QuantStub)")
        lead = x.shape[:-2] if nd >= 2 else x.shape[:-1]
        H = x.shape[-2] if nd >= 2 else 1
        W = x.shape[-1]
        (pt, pb) = pads[-2] if nd >= 2 else (0, 0)
        (pl, pr) = pads[-1]
        padded = Tensor.empty((*lead, *( [H + pt + pb] if nd >= 2 else []), W + pl + pr), T.float32, "hip")
        _C.call("lq_pad_planes_f32", x.data_ptr, padded.data_ptr, int(np.prod(lead, dtype=np.int64)), H, W, pt, pb,
                pl, pr, mode, None)
        x, conv_pad = padded, (0,) * nd
    if nd == 1:
        y = F.conv1d_f32(x, w, mod.bias, mod.stride[-1], conv_pad[0], mod.dilation[-1], mod.groups)
    elif nd == 2:
        y = F.conv2d_f32(x, w, mod.bias, mod.stride, conv_pad, mod.dilation, mod.groups)
    else:
        y = F.conv3d_f32(x, w, mod.bias, mod.stride, conv_pad, mod.dilation, mod.groups)
    if relu:
        _C.call("lq_relu_f32", y.data_ptr, y.data_ptr, y.numel, None)
    q = mod.__dict__.get("_out_quantize")
    if q is None:
        q = Quantize(mod.scale, mod.zero_point, mod.out_qdtype)
        mod.__dict__["_out_quantize"] = q
    return q(y)


def input_grid(x: Tensor, what: str) -> Grid:
    if not isinstance(x, Tensor) or x.device != "hip":
        raise _C.DeviceMismatch(f"{what}: input must be a tensor on the 'hip' device")
    if x._grid is None:
        raise NotImplementedError(
            f"{what}: the input is a plain float tensor, not an activation on a quantization "
            "grid. Feed it through nn.quantized.Quantize (QuantStub) first; the float-input "
            "form of this layer is Lucid's dequantize-to-float path, which this backend does "
            "not provide.")
    return x._grid


def plain_volume_grid(x: Tensor, g: Grid) -> Grid:
    """The grid of a 5-d activation with its codes in (B, C, D, H, W) order: channels-last
    codes (layout "nhwc", what the volumetric convolution leaves) are transposed back."""
    if g.layout == "plain":
        return g
    B, Cc = x.shape[0], x.shape[1]
    vol = x.numel // max(B * Cc, 1)
    codes = Tensor.empty(x.shape, T.int8, "hip")
    _C.call("lq_transpose_i8", g.codes.data_ptr, codes.data_ptr, B, vol, Cc, vol * Cc, Cc * vol, None)
    return Grid(codes, g.scale, g.zero_point, g.qdtype, g.offset, g.zp_host, "plain")


def zp_args(g: Grid) -> tuple[int, Tensor | None]:
    """``(a_zp, a_zp_dev)`` for the GEMM / conv entry points: a host zero point
    when it is known, otherwise the device scalar plus the storage offset."""
    if g.zp_host is not None:
        return int(g.zp_host) + g.offset, None
    return g.offset, g.zero_point


def host_scalar(t: Tensor) -> float:
    return float(t.numpy().reshape(-1)[0])
