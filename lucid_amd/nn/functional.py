"""float32 functional ops that sit between the quantized Linears of a
transformer block (``lucid.nn.functional``: ``layer_norm``, ``gelu``,
``scaled_dot_product_attention``) plus the residual add.  Each is one HIP
kernel; inputs and outputs are float32 tensors on the ``hip`` device.
"""

from __future__ import annotations

import math

from .. import _C
from .. import _tensor as T
from .._tensor import Tensor


def _require_f32_hip(name: str, *ts: Tensor) -> None:
    for t in ts:
        if not isinstance(t, Tensor) or t.device != "hip":
            raise _C.DeviceMismatch(f"{name}: inputs must be tensors on the 'hip' device")
        if t.dtype != T.float32:
            raise _C.DtypeMismatch(f"{name} expects float32, got {t.dtype}")


def _new_range() -> Tensor:
    """Device buffer into which a kernel stores the per-block min / max of the
    tensor it is about to write (``lq_range_buffer_bytes``)."""
    _C.init()
    return Tensor.empty((_C.range_buffer_words(),), T.float32, "hip")


def layer_norm(x: Tensor, normalized_shape, weight: Tensor, bias: Tensor, eps: float = 1e-5,
               track_range: bool = False) -> Tensor:
    """``F.layer_norm`` over the last axis (``lucid/_C/backend/cpu/Norm.cpp:35-65``).
    ``track_range`` makes the kernel keep the min / max of its output, which a
    dynamic-quantized Linear fed with the result then uses instead of a pass of
    its own (same for ``gelu`` and the attention below)."""
    _require_f32_hip("layer_norm", x, weight, bias)
    cols = normalized_shape if isinstance(normalized_shape, int) else int(normalized_shape[-1])
    if x.shape[-1] != cols or weight.numel != cols or bias.numel != cols:
        raise _C.ShapeMismatch(f"layer_norm: last dim {x.shape[-1]} vs normalized_shape {cols}")
    out = Tensor.empty(x.shape, T.float32, "hip")
    out._range = _new_range() if track_range else None
    _C.call("lq_layernorm_f32", x.data_ptr, weight.data_ptr, bias.data_ptr, out.data_ptr,
            x.numel // cols, cols, float(eps), out._range.data_ptr if track_range else None, None)
    return out


def layer_norm_dynamic_quantize(x: Tensor, normalized_shape, weight: Tensor, bias: Tensor, eps: float, qdtype):
    """``layer_norm`` followed by the per-tensor affine dynamic quantization of a
    dynamic-quantized Linear (``dynamic/linear.py:87-92``), without storing the float32
    result: ``(codes [rows, cols] int8, scale, zero_point)`` - the bits that ``layer_norm(...,
    track_range=True)`` and the Linear's own quantization produce.  ``None`` when the rows are
    not what the fused kernels take (the caller then takes the two-step route)."""
    _require_f32_hip("layer_norm", x, weight, bias)
    cols = normalized_shape if isinstance(normalized_shape, int) else int(normalized_shape[-1])
    if x.shape[-1] != cols or weight.numel != cols or bias.numel != cols:
        raise _C.ShapeMismatch(f"layer_norm: last dim {x.shape[-1]} vs normalized_shape {cols}")
    rows = x.numel // cols
    if cols % 4 or cols > 2048 or rows == 0 or (rows + 3) // 4 > 16384:
        return None
    from .quantized._utils import storage_offset
    stats = Tensor.empty((rows, 2), T.float32, "hip")
    rng = _new_range()
    _C.call("lq_layernorm_stats_f32", x.data_ptr, weight.data_ptr, bias.data_ptr, rows, cols, float(eps),
            stats.data_ptr, rng.data_ptr, None)
    scale, zp = Tensor.empty((), T.float32, "hip"), Tensor.empty((), T.float32, "hip")
    _C.call("lq_calc_qparams_from_range", rng.data_ptr, 0, qdtype.quant_min, qdtype.quant_max, int(qdtype.signed),
            1e-8, scale.data_ptr, zp.data_ptr, None, None, None)
    q = Tensor.empty((rows, cols), T.int8, "hip")
    _C.call("lq_layernorm_quantize_i8", x.data_ptr, weight.data_ptr, bias.data_ptr, stats.data_ptr, rows, cols,
            scale.data_ptr, zp.data_ptr, qdtype.quant_min, qdtype.quant_max, storage_offset(qdtype), q.data_ptr, None)
    return q, scale, zp


def gelu(x: Tensor, approximate: str = "none", track_range: bool = False) -> Tensor:
    """``F.gelu`` (``lucid/nn/functional/activations.py:219``), exact erf form."""
    if approximate != "none":
        raise NotImplementedError("gelu: only approximate='none' is built")
    _require_f32_hip("gelu", x)
    out = Tensor.empty(x.shape, T.float32, "hip")
    out._range = _new_range() if track_range else None
    _C.call("lq_gelu_f32", x.data_ptr, out.data_ptr, x.numel, out._range.data_ptr if track_range else None,
            None)
    return out


def add(a: Tensor, b: Tensor) -> Tensor:
    _require_f32_hip("add", a, b)
    if a.shape != b.shape:
        raise _C.ShapeMismatch(f"add: {a.shape} vs {b.shape}")
    out = Tensor.empty(a.shape, T.float32, "hip")
    _C.call("lq_add_f32", a.data_ptr, b.data_ptr, out.data_ptr, a.numel, None)
    return out


def scaled_dot_product_attention_qkv(qkv: Tensor, num_heads: int, scale: float | None = None,
                                     track_range: bool = False) -> Tensor:
    """``F.scaled_dot_product_attention(q, k, v)`` on the packed output of a qkv
    Linear: ``qkv`` is ``(B, T, 3*H*D)`` laid out ``(B, T, 3, H, D)`` as in
    ``lucid/models/vision/vit/_model.py:137-141``; returns ``(B, T, H*D)``, the
    ``permute(0, 2, 1, 3).reshape(B, T, C)`` of ``_model.py:158``."""
    _require_f32_hip("scaled_dot_product_attention", qkv)
    if qkv.ndim != 3 or qkv.shape[2] % (3 * num_heads):
        raise _C.ShapeMismatch(f"attention: bad packed qkv shape {qkv.shape} for {num_heads} heads")
    B, Tn, C3 = qkv.shape
    D = C3 // (3 * num_heads)
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    out = Tensor.empty((B, Tn, num_heads * D), T.float32, "hip")
    out._range = _new_range() if track_range else None
    _C.call("lq_attention_f32", qkv.data_ptr, out.data_ptr, B, Tn, num_heads, D, s,
            out._range.data_ptr if track_range else None, None)
    return out


def conv2d_f32(x: Tensor, weight: Tensor, bias: Tensor | None = None, stride=(1, 1), padding=(0, 0),
               dilation=(1, 1), groups: int = 1) -> Tensor:
    """``F.conv2d`` in float32 with zero padding (``CpuBackend.h:8124-8257``): NCHW input, OIHW
    weight, symmetric ``padding`` = (h, w).  Calibration and QAT forwards only."""
    _require_f32_hip("conv2d", x, weight)
    if x.ndim != 4 or weight.ndim != 4 or weight.shape[1] * groups != x.shape[1]:
        raise _C.ShapeMismatch(f"conv2d: input {x.shape} and weight {weight.shape} (groups={groups}) do not match")
    B, Cin, H, W = x.shape
    Cout, _, KH, KW = weight.shape
    OH = (H + 2 * padding[0] - dilation[0] * (KH - 1) - 1) // stride[0] + 1
    OW = (W + 2 * padding[1] - dilation[1] * (KW - 1) - 1) // stride[1] + 1
    out = Tensor.empty((B, Cout, max(OH, 0), max(OW, 0)), T.float32, "hip")
    _C.call("lq_conv2d_f32", x.data_ptr, weight.data_ptr, bias.data_ptr if bias is not None else None, out.data_ptr,
            B, Cin, H, W, Cout, KH, KW, int(stride[0]), int(stride[1]), int(padding[0]), int(padding[1]),
            int(dilation[0]), int(dilation[1]), int(groups), None)
    return out


def conv1d_f32(x: Tensor, weight: Tensor, bias: Tensor | None = None, stride: int = 1, padding: int = 0,
               dilation: int = 1, groups: int = 1) -> Tensor:
    """``F.conv1d`` in float32: the 2-d kernel on a one-row image."""
    _require_f32_hip("conv1d", x, weight)
    if x.ndim != 3 or weight.ndim != 3:
        raise _C.ShapeMismatch(f"conv1d: expected (B, C, L) input and (O, I, K) weight, got {x.shape} and {weight.shape}")
    B, Cc, Ln = x.shape
    O, I, K = weight.shape
    y = conv2d_f32(x.reshape(B, Cc, 1, Ln), weight.reshape(O, I, 1, K), bias, (1, int(stride)), (0, int(padding)),
                   (1, int(dilation)), groups)
    return y.reshape(B, O, y.shape[3])


def conv3d_f32(x: Tensor, weight: Tensor, bias: Tensor | None = None, stride=(1, 1, 1), padding=(0, 0, 0),
               dilation=(1, 1, 1), groups: int = 1) -> Tensor:
    """``F.conv3d`` in float32 with zero padding, for calibration and QAT forwards of volumetric
    models: every output depth slice is the sum over the kernel's depth taps of a 2-d convolution
    of one input depth slice (pitched device copies cut the slices out of ``(B, C, D, H, W)``).
    The summation order differs from Lucid's im2col GEMM, so the result agrees with it to
    float32 rounding, not bit for bit."""
    _require_f32_hip("conv3d", x, weight)
    if x.ndim != 5 or weight.ndim != 5 or weight.shape[1] * groups != x.shape[1]:
        raise _C.ShapeMismatch(f"conv3d: input {x.shape} and weight {weight.shape} (groups={groups}) do not match")
    B, Cin, D, H, W = x.shape
    Cout, Cg, KD, KH, KW = weight.shape
    (sd, sh, sw), (pd, ph, pw), (dd, dh, dw) = stride, padding, dilation
    OD = (D + 2 * pd - dd * (KD - 1) - 1) // sd + 1
    OH = (H + 2 * ph - dh * (KH - 1) - 1) // sh + 1
    OW = (W + 2 * pw - dw * (KW - 1) - 1) // sw + 1
    if min(OD, OH, OW) < 1:
        raise _C.ShapeMismatch(f"conv3d: kernel {(KD, KH, KW)} does not fit input {x.shape}")
    out = Tensor.empty((B, Cout, OD, OH, OW), T.float32, "hip")
    # the kernel's depth taps as KD contiguous (Cout, Cg, KH, KW) filters
    taps = []
    for kd in range(KD):
        wk = Tensor.empty((Cout, Cg, KH, KW), T.float32, "hip")
        _C.call("lq_d2d_rows", wk.data_ptr, KH * KW * 4, weight.data_ptr + kd * KH * KW * 4, KD * KH * KW * 4,
                KH * KW * 4, Cout * Cg, None)
        taps.append(wk)
    plane_in, plane_out = H * W * 4, OH * OW * 4
    xs = Tensor.empty((B, Cin, H, W), T.float32, "hip")
    for od in range(OD):
        acc = None
        for kd in range(KD):
            z = od * sd - pd + kd * dd
            if z < 0 or z >= D:
                continue  # a tap in the zero padding
            _C.call("lq_d2d_rows", xs.data_ptr, plane_in, x.data_ptr + z * plane_in, D * plane_in, plane_in, B * Cin, None)
            part = conv2d_f32(xs, taps[kd], None, (sh, sw), (ph, pw), (dh, dw), groups)
            if acc is None:
                acc = part
            else:
                _C.call("lq_add_f32", acc.data_ptr, part.data_ptr, acc.data_ptr, acc.numel, None)
        if acc is None:
            acc = Tensor.empty((B, Cout, OH, OW), T.float32, "hip")
            _C.call("lq_fill_bytes", acc.data_ptr, 0, acc.nbytes, None)
        if bias is not None:
            # y[b, c, :, :] + bias[c]: the bias as a (B * Cout, OH * OW) broadcast
            full = Tensor.empty(acc.shape, T.float32, "hip")
            _C.call("lq_broadcast_f32", bias.data_ptr, full.data_ptr, B, Cout, OH * OW, None)
            _C.call("lq_add_f32", acc.data_ptr, full.data_ptr, acc.data_ptr, acc.numel, None)
        _C.call("lq_d2d_rows", out.data_ptr + od * plane_out, OD * plane_out, acc.data_ptr, plane_out, plane_out,
                B * Cout, None)
    return out


def linear_f32(x: Tensor, weight: Tensor, bias: Tensor | None = None) -> Tensor:
    """``F.linear`` in float32 (``CpuBackend.h:4525``): ``x @ weight.T + bias``."""
    _require_f32_hip("linear", x, weight)
    K = weight.shape[1]
    if x.shape[-1] != K:
        raise _C.ShapeMismatch(f"linear: {x.shape} @ {weight.shape}^T")
    M, N = x.numel // K, weight.shape[0]
    out = Tensor.empty((*x.shape[:-1], N), T.float32, "hip")
    _C.call("lq_sgemm_nt_f32", x.data_ptr, weight.data_ptr, bias.data_ptr if bias is not None else None,
            out.data_ptr, M, N, K, None)
    return out
