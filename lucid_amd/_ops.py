"""Thin argument marshalling for the fused GEMM / conv entry points.

These helpers only fill the C structs of ``include/lucid_hip.h`` from
``Tensor`` handles and validate devices; the quantized modules build on them.
"""

from __future__ import annotations

import ctypes as C

from . import _C
from . import _tensor as T
from ._tensor import Tensor

OUT_ACC_I32, OUT_F32, OUT_F16, OUT_REQUANT_I8, OUT_FAKEQUANT_F32 = range(5)
_OUT_DTYPE = {OUT_ACC_I32: T.int32, OUT_F32: T.float32, OUT_F16: T.float16,
              OUT_REQUANT_I8: T.int8, OUT_FAKEQUANT_F32: T.float32}
PATH_AUTO, PATH_TILE, PATH_SKINNY, PATH_NAIVE = range(4)


def _ptr(t: Tensor | None, what: str, dt=None):
    if t is None:
        return None
    if not isinstance(t, Tensor) or t.device != "hip":
        raise _C.DeviceMismatch(f"{what} must be a tensor on the 'hip' device")
    if dt is not None and t.dtype not in (dt if isinstance(dt, tuple) else (dt,)):
        raise _C.DtypeMismatch(f"{what} has dtype {t.dtype}, expected {dt}")
    return t.data_ptr


def rowsum_i8(w: Tensor) -> Tensor:
    """``sum_k w[n, k]`` as int32, over everything but the first axis."""
    N = w.shape[0]
    K = w.numel // max(N, 1)
    out = Tensor.empty((N,), T.int32, "hip")
    _C.call("lq_rowsum_i8", _ptr(w, "w", T.int8), out.data_ptr, N, K, None)
    return out


def qlinear_i8(a: Tensor, w: Tensor, *, a_zp: int = 0, a_zp_dev: Tensor | None = None,
               a_scale: Tensor | None = None,
               w_scale: Tensor | None = None, wsum: Tensor | None = None,
               bias: Tensor | None = None, relu: bool = False, out_mode: int = OUT_F32,
               out_scale: Tensor | None = None, out_zp: Tensor | None = None, out_qmin: int = 0,
               out_qmax: int = 255, out_offset: int = 0, path: int = PATH_AUTO,
               tile_config: int = 0, out: Tensor | None = None, repeat: int = 1,
               residual: Tensor | None = None, join=None, gelu: bool = False,
               range_buf: Tensor | None = None, w_zp: Tensor | None = None) -> Tensor:
    """Fused int8 GEMM + epilogue; see ``lq_qlinear_i8`` in ``lucid_hip.h``.
    ``a`` is int8 ``[M, K]``, ``w`` int8 ``[N, K]``; the result is ``[M, N]``.
    ``w_zp`` (int32 ``[N]``) holds the zero points of affine weight rows.
    ``residual`` (float32, ``M*N`` elements) is added after the activation;
    ``join`` fuses a residual add on codes after the requantize (see ``_fill_join``)."""
    if a.ndim != 2 or w.ndim != 2 or a.shape[1] != w.shape[1]:
        raise _C.ShapeMismatch(f"qlinear_i8: a {a.shape} and w {w.shape} do not form a GEMM")
    M, K = a.shape
    N = w.shape[0]
    if out is None:
        out = Tensor.empty((M, N), _OUT_DTYPE[out_mode], "hip")
    args = _C.QLinearArgs()
    args.a, args.w = _ptr(a, "a", T.int8), _ptr(w, "w", T.int8)
    args.M, args.N, args.K = M, N, K
    args.wsum = _ptr(wsum, "wsum", T.int32)
    args.a_zp = int(a_zp)
    args.a_zp_dev = _ptr(a_zp_dev, "a_zp_dev", T.float32)
    args.a_scale = _ptr(a_scale, "a_scale", T.float32)
    args.a_scale_per_row = int(a_scale is not None and a_scale.numel != 1)
    if a_scale is not None and a_scale.numel not in (1, M):
        raise _C.ShapeMismatch(f"a_scale has {a_scale.numel} entries for M = {M}")
    if w_scale is not None and w_scale.numel != N:
        raise _C.ShapeMismatch(f"w_scale has {w_scale.numel} entries for N = {N}")
    args.w_scale = _ptr(w_scale, "w_scale", T.float32)
    args.bias = _ptr(bias, "bias", (T.float32, T.float16))
    args.bias_dtype = bias.dtype.code if bias is not None else 0
    if bias is not None and bias.numel != N:
        raise _C.ShapeMismatch(f"bias has {bias.numel} entries for N = {N}")
    args.relu, args.out_mode = int(relu), int(out_mode)
    args.out_scale = _ptr(out_scale, "out_scale", T.float32)
    args.out_zp = _ptr(out_zp, "out_zp", T.float32)
    args.out_qmin, args.out_qmax, args.out_offset = int(out_qmin), int(out_qmax), int(out_offset)
    args.out, args.ldo, args.force_path = out.data_ptr, 0, int(path)
    args.tile_config = int(tile_config)
    if residual is not None and residual.numel != M * N:
        raise _C.ShapeMismatch(f"residual has {residual.numel} elements for an output of {M}x{N}")
    args.residual, args.ldr = _ptr(residual, "residual", T.float32), 0
    _fill_join(args.join, join, (M, N))
    args.gelu, args.range = int(gelu), _ptr(range_buf, "range", T.float32)
    if w_zp is not None and w_zp.numel != N:
        raise _C.ShapeMismatch(f"w_zp has {w_zp.numel} entries for N = {N}")
    args.w_zp = _ptr(w_zp, "w_zp", T.int32)
    if repeat == 1:
        _C.call("lq_qlinear_i8", C.byref(args), None)
    else:
        _C.call("lq_qlinear_i8_n", C.byref(args), int(repeat), None)
    return out


CONV_AUTO, CONV_GEMM, CONV_IMPLICIT, CONV_IM2COL, CONV_NAIVE, CONV_PACKED4, CONV_PREPACKED4 = range(7)


def conv_out_size(size: int, k: int, stride: int, pad_lo: int, pad_hi: int, dil: int) -> int:
    """Output extent of one spatial axis (``lucid/_C/nn/ConvNd.cpp:56-59``)."""
    return (size + pad_lo + pad_hi - dil * (k - 1) - 1) // stride + 1


def _fill_join(j, join, out_shape) -> None:
    """``join`` = dict(q=codes tensor shaped like the output, offset, scale, zp, relu, out_scale,
    out_zp, out_qmin, out_qmax, out_offset): the residual add on codes fused into the epilogue."""
    if join is None:
        return
    q = join["q"]
    if tuple(q.shape) != tuple(out_shape):
        raise _C.ShapeMismatch(f"join operand {q.shape} does not match the output {tuple(out_shape)}")
    j.q, j.ld, j.offset = _ptr(q, "join.q", T.int8), 0, int(join["offset"])
    j.scale, j.zp = _ptr(join["scale"], "join.scale", T.float32), _ptr(join["zp"], "join.zp", T.float32)
    j.relu = int(join.get("relu", False))
    j.out_scale = _ptr(join["out_scale"], "join.out_scale", T.float32)
    j.out_zp = _ptr(join["out_zp"], "join.out_zp", T.float32)
    j.out_qmin, j.out_qmax, j.out_offset = int(join["out_qmin"]), int(join["out_qmax"]), int(join["out_offset"])


def qconv2d_i8(x: Tensor, w: Tensor, *, a_zp: int, a_scale: Tensor | None = None,
               w_scale: Tensor | None = None, wsum: Tensor | None = None,
               bias: Tensor | None = None, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1),
               groups: int = 1, relu: bool = False, out_mode: int = OUT_F32,
               out_scale: Tensor | None = None, out_zp: Tensor | None = None, out_qmin: int = 0,
               out_qmax: int = 255, out_offset: int = 0, path: int = CONV_AUTO,
               tile_config: int = 0, join=None, w_zp: Tensor | None = None,
               logical: tuple[int, int, int, int] | None = None) -> Tensor:
    """Fused int8 convolution; see ``lq_qconv2d_i8``.  ``x`` int8 NHWC, ``w``
    int8 ``[Cout, KH, KW, Cin/groups]``, ``pad`` = (h_lo, h_hi, w_lo, w_hi);
    ``w_zp`` (int32 ``[Cout]``) holds the zero points of affine filters.
    With ``path=CONV_PREPACKED4`` ``x`` and ``w`` are the packed tensors of
    ``quantize_nchw_to_packed4`` and ``pack4_filter_i8`` and ``logical`` = (H, W, Cin, KW)
    of the layer they stand for.  Returns NHWC ``[B, OH, OW, Cout]``."""
    if x.ndim != 4 or w.ndim != 4:
        raise _C.ShapeMismatch(f"qconv2d_i8: expected 4-d x and w, got {x.shape} and {w.shape}")
    if path == CONV_PREPACKED4:
        if logical is None or groups != 1:
            raise ValueError("qconv2d_i8: packed operands need logical=(H, W, Cin, KW) and groups == 1")
        H, W, Cin, KW = (int(v) for v in logical)
        Hp, Wp, KWp = packed4_geometry(H, W, Cin, KW, int(stride[1]), pad)
        B, Cout, KH = x.shape[0], w.shape[0], w.shape[1]
        if tuple(x.shape[1:]) != (Hp, Wp, 4) or tuple(w.shape[2:]) != (KWp, 4):
            raise _C.ShapeMismatch(f"qconv2d_i8: packed x {x.shape} / w {w.shape} do not match the layer's "
                                   f"[B, {Hp}, {Wp}, 4] / [Cout, KH, {KWp}, 4]")
    else:
        B, H, W, Cin = x.shape
        Cout, KH, KW, Cg = w.shape
        if Cg * groups != Cin:
            raise _C.ShapeMismatch(f"qconv2d_i8: weight {w.shape} does not match Cin={Cin}, groups={groups}")
    OH = conv_out_size(H, KH, stride[0], pad[0], pad[1], dilation[0])
    OW = conv_out_size(W, KW, stride[1], pad[2], pad[3], dilation[1])
    out = Tensor.empty((B, max(OH, 0), max(OW, 0), Cout), _OUT_DTYPE[out_mode], "hip")
    a = _C.QConv2dArgs()
    a.x, a.w = _ptr(x, "x", T.int8), _ptr(w, "w", T.int8)
    a.B, a.H, a.W, a.Cin, a.Cout, a.KH, a.KW = B, H, W, Cin, Cout, KH, KW
    a.stride_h, a.stride_w = int(stride[0]), int(stride[1])
    a.pad_h_lo, a.pad_h_hi, a.pad_w_lo, a.pad_w_hi = (int(v) for v in pad)
    a.dil_h, a.dil_w, a.groups = int(dilation[0]), int(dilation[1]), int(groups)
    a.wsum, a.a_zp = _ptr(wsum, "wsum", T.int32), int(a_zp)
    a.a_scale, a.w_scale = _ptr(a_scale, "a_scale", T.float32), _ptr(w_scale, "w_scale", T.float32)
    a.bias = _ptr(bias, "bias", (T.float32, T.float16))
    a.bias_dtype = bias.dtype.code if bias is not None else 0
    a.relu, a.out_mode = int(relu), int(out_mode)
    a.out_scale, a.out_zp = _ptr(out_scale, "out_scale", T.float32), _ptr(out_zp, "out_zp", T.float32)
    a.out_qmin, a.out_qmax, a.out_offset = int(out_qmin), int(out_qmax), int(out_offset)
    a.out, a.force_path, a.tile_config = out.data_ptr, int(path), int(tile_config)
    _fill_join(a.join, join, out.shape)
    if w_zp is not None and w_zp.numel != Cout:
        raise _C.ShapeMismatch(f"w_zp has {w_zp.numel} entries for Cout = {Cout}")
    a.w_zp = _ptr(w_zp, "w_zp", T.int32)
    _C.call("lq_qconv2d_i8", C.byref(a), None)
    return out


def packed4_geometry(H: int, W: int, Cin: int, KW: int, stride_w: int, pad) -> tuple[int, int, int]:
    """(Hp, Wp, KWp) of the packed four-channel image and filter of a layer with at most four
    input channels; see ``lq_qconv2d_packed4_geometry``."""
    a = _C.QConv2dArgs()
    a.H, a.W, a.Cin, a.KW, a.KH, a.B, a.Cout = int(H), int(W), int(Cin), int(KW), 1, 1, 1
    a.stride_h, a.stride_w, a.dil_h, a.dil_w, a.groups = 1, int(stride_w), 1, 1, 1
    a.pad_h_lo, a.pad_h_hi, a.pad_w_lo, a.pad_w_hi = (int(v) for v in pad)
    hp, wp, kwp = C.c_int(), C.c_int(), C.c_int()
    _C.call("lq_qconv2d_packed4_geometry", C.byref(a), C.byref(hp), C.byref(wp), C.byref(kwp))
    return hp.value, wp.value, kwp.value


def quantize_nchw_to_packed4(x: Tensor, scale: Tensor, zero_point: Tensor, qmin: int, qmax: int, offset: int,
                             fill_code: int, pad, Hp: int, Wp: int) -> Tensor:
    """float32 NCHW (C <= 4) -> int8 ``[B, Hp, Wp, 4]`` codes of the few-channel convolution
    route; see ``lq_quantize_nchw_to_packed4``."""
    if x.ndim != 4 or x.dtype != T.float32:
        raise _C.ShapeMismatch(f"quantize_nchw_to_packed4: expected a float32 (B, C, H, W) tensor, got {x.shape}")
    B, Cc, H, W = x.shape
    out = Tensor.empty((B, Hp, Wp, 4), T.int8, "hip")
    _C.call("lq_quantize_nchw_to_packed4", _ptr(x, "x", T.float32), out.data_ptr, int(offset), B, Cc, H, W,
            int(pad[0]), int(pad[2]), int(Hp), int(Wp), _ptr(scale, "scale", T.float32),
            _ptr(zero_point, "zero_point", T.float32), int(qmin), int(qmax), int(fill_code), None)
    return out


def pack4_filter_i8(w: Tensor) -> Tensor:
    """int8 ``[Cout, KH, KW, Cin]`` (Cin <= 4) -> ``[Cout, KH, KWp, 4]`` with zeros in the added
    taps and channels; see ``lq_pack4_filter_i8``."""
    Cout, KH, KW, Cin = w.shape
    out = Tensor.empty((Cout, KH, (KW + 3) // 4 * 4, 4), T.int8, "hip")
    _C.call("lq_pack4_filter_i8", _ptr(w, "w", T.int8), out.data_ptr, Cout, KH, KW, Cin, None)
    return out


def qconv3d_i8(x: Tensor, w: Tensor, *, a_zp: int, a_scale: Tensor | None = None,
               w_scale: Tensor | None = None, wsum: Tensor | None = None, bias: Tensor | None = None,
               stride=(1, 1, 1), pad=((0, 0),) * 3, dilation=(1, 1, 1), groups: int = 1, relu: bool = False,
               out_mode: int = OUT_F32, out_scale: Tensor | None = None, out_zp: Tensor | None = None,
               out_qmin: int = 0, out_qmax: int = 255, out_offset: int = 0, tile_config: int = 0,
               w_zp: Tensor | None = None) -> Tensor:
    """Fused int8 volumetric convolution; see ``lq_qconv3d_i8``.  ``x`` int8 NDHWC, ``w`` int8
    ``[Cout, KD, KH, KW, Cin/groups]``, ``pad`` = ((lo, hi),) * 3 for depth, height, width.
    Returns NDHWC ``[B, OD, OH, OW, Cout]``."""
    if x.ndim != 5 or w.ndim != 5:
        raise _C.ShapeMismatch(f"qconv3d_i8: expected 5-d x and w, got {x.shape} and {w.shape}")
    B, D, H, W, Cin = x.shape
    Cout, KD, KH, KW, Cg = w.shape
    if Cg * groups != Cin:
        raise _C.ShapeMismatch(f"qconv3d_i8: weight {w.shape} does not match Cin={Cin}, groups={groups}")
    outs = [conv_out_size(n, k, int(s), int(lo), int(hi), int(d))
            for n, k, s, (lo, hi), d in zip((D, H, W), (KD, KH, KW), stride, pad, dilation)]
    out = Tensor.empty((B, *[max(o, 0) for o in outs], Cout), _OUT_DTYPE[out_mode], "hip")
    a = _C.QConv3dArgs()
    a.x, a.w = _ptr(x, "x", T.int8), _ptr(w, "w", T.int8)
    a.B, a.D, a.H, a.W, a.Cin, a.Cout, a.KD, a.KH, a.KW = B, D, H, W, Cin, Cout, KD, KH, KW
    for i in range(3):
        a.stride[i], a.dilation[i] = int(stride[i]), int(dilation[i])
        a.pad_lo[i], a.pad_hi[i] = int(pad[i][0]), int(pad[i][1])
    a.groups = int(groups)
    a.wsum, a.a_zp = _ptr(wsum, "wsum", T.int32), int(a_zp)
    a.a_scale, a.w_scale = _ptr(a_scale, "a_scale", T.float32), _ptr(w_scale, "w_scale", T.float32)
    a.bias = _ptr(bias, "bias", (T.float32, T.float16))
    a.bias_dtype = bias.dtype.code if bias is not None else 0
    a.relu, a.out_mode = int(relu), int(out_mode)
    a.out_scale, a.out_zp = _ptr(out_scale, "out_scale", T.float32), _ptr(out_zp, "out_zp", T.float32)
    a.out_qmin, a.out_qmax, a.out_offset = int(out_qmin), int(out_qmax), int(out_offset)
    a.out, a.tile_config = out.data_ptr, int(tile_config)
    if w_zp is not None and w_zp.numel != Cout:
        raise _C.ShapeMismatch(f"w_zp has {w_zp.numel} entries for Cout = {Cout}")
    a.w_zp = _ptr(w_zp, "w_zp", T.int32)
    _C.call("lq_qconv3d_i8", C.byref(a), None)
    return out
