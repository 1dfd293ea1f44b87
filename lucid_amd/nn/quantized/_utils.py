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
