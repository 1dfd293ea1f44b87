"""numpy front-end of the CPU oracle (``lucid_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The product package never
imports this module.

Every wrapper takes and returns numpy arrays and forwards to the C function of
the same name; see the C file for the reference citations.
"""

from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblucid_oracle.so")

I8, I16 = 1, 2
OUT_ACC_I32, OUT_F32, OUT_F16, OUT_REQUANT_I8, OUT_FAKEQUANT_F32 = 0, 1, 2, 3, 4
BIAS_NONE, BIAS_F16, BIAS_F32 = 0, 5, 6


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f32_to_f16.restype = C.c_uint16
        _lib.orc_f32_to_f16.argtypes = [C.c_float]
        _lib.orc_f16_to_f32.restype = C.c_float
        _lib.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_conv_out_size.restype = C.c_int
    return _lib


def set_threads(n: int = 0) -> int:
    """Set (n > 0) and return the OpenMP thread count the oracle's loops use."""
    return int(lib().orc_set_threads(int(n)))


def _p(a: np.ndarray | None):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ocl(shape, ch_axis):
    """(outer, C, inner) extents of a contiguous tensor around ``ch_axis``."""
    if ch_axis is None:
        return 1, 1, int(np.prod(shape, dtype=np.int64))
    ch_axis %= len(shape)
    outer = int(np.prod(shape[:ch_axis], dtype=np.int64))
    inner = int(np.prod(shape[ch_axis + 1 :], dtype=np.int64))
    return outer, int(shape[ch_axis]), inner


def _qp(scale, zp, Cn):
    s = np.ascontiguousarray(np.broadcast_to(_f32(scale).reshape(-1), (Cn,)))
    z = np.ascontiguousarray(np.broadcast_to(_f32(zp).reshape(-1), (Cn,)))
    return s, z


def _code_np(q_dtype):
    return np.int8 if q_dtype == I8 else np.int16


def quantize(x, scale, zp, qmin, qmax, ch_axis=None, q_dtype=I8, code_offset=0, faithful=False):
    x = _f32(x)
    o, c, i = _ocl(x.shape, ch_axis)
    s, z = _qp(scale, zp, c)
    q = np.empty(x.shape, dtype=_code_np(q_dtype))
    sz = C.c_size_t
    if faithful:
        assert code_offset == 0
        lib().orc_quantize_faithful(_p(x), _p(q), q_dtype, sz(o), sz(c), sz(i), _p(s), _p(z),
                                    int(qmin), int(qmax))
    else:
        lib().orc_quantize(_p(x), _p(q), q_dtype, int(code_offset), sz(o), sz(c), sz(i), _p(s),
                           _p(z), int(qmin), int(qmax))
    return q


def dequantize(q, scale, zp, ch_axis=None, code_offset=0, faithful=False):
    q = np.ascontiguousarray(q)
    q_dtype = {np.dtype(np.int8): I8, np.dtype(np.int16): I16}[q.dtype]
    o, c, i = _ocl(q.shape, ch_axis)
    s, z = _qp(scale, zp, c)
    out = np.empty(q.shape, dtype=np.float32)
    sz = C.c_size_t
    if faithful:
        assert code_offset == 0
        lib().orc_dequantize_faithful(_p(q), q_dtype, _p(out), sz(o), sz(c), sz(i), _p(s), _p(z))
    else:
        lib().orc_dequantize(_p(q), q_dtype, int(code_offset), _p(out), sz(o), sz(c), sz(i),
                             _p(s), _p(z))
    return out


def fake_quantize(x, scale, zp, qmin, qmax, ch_axis=None, faithful=False):
    x = _f32(x)
    o, c, i = _ocl(x.shape, ch_axis)
    s, z = _qp(scale, zp, c)
    out = np.empty(x.shape, dtype=np.float32)
    sz = C.c_size_t
    fn = lib().orc_fake_quantize_faithful if faithful else lib().orc_fake_quantize
    fn(_p(x), _p(out), sz(o), sz(c), sz(i), _p(s), _p(z), int(qmin), int(qmax))
    return out


def minmax(x, ch_axis=None):
    x = _f32(x)
    o, c, i = _ocl(x.shape, ch_axis)
    mn = np.empty(c, dtype=np.float32)
    mx = np.empty(c, dtype=np.float32)
    sz = C.c_size_t
    lib().orc_minmax(_p(x), sz(o), sz(c), sz(i), _p(mn), _p(mx))
    return mn, mx


def calc_qparams(mn, mx, symmetric, qmin, qmax, signed, eps=1e-8):
    mn = _f32(mn).reshape(-1)
    mx = _f32(mx).reshape(-1)
    n = mn.size
    s = np.empty(n, dtype=np.float32)
    z = np.empty(n, dtype=np.float32)
    lib().orc_calc_qparams(_p(mn), _p(mx), C.c_size_t(n), int(bool(symmetric)), int(qmin),
                           int(qmax), int(bool(signed)), C.c_float(eps), _p(s), _p(z))
    return s, z


def f32_to_f16_bits(x):
    x = _f32(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_f32_to_f16_array(_p(x), _p(out), C.c_size_t(x.size))
    return out


def igemm(a, w):
    a = np.ascontiguousarray(a, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = a.shape
    N, K2 = w.shape
    assert K == K2
    acc = np.empty((M, N), dtype=np.int32)
    lib().orc_igemm(_p(a), _p(w), _p(acc), M, N, K)
    return acc


def igemm_a16(a, w):
    a = np.ascontiguousarray(a, dtype=np.int16)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = a.shape
    N, _ = w.shape
    acc = np.empty((M, N), dtype=np.int64)
    lib().orc_igemm_a16(_p(a), _p(w), _p(acc), M, N, K)
    return acc


def rowsum_i8(w):
    w = np.ascontiguousarray(w, dtype=np.int8)
    w2 = w.reshape(w.shape[0], -1)
    out = np.empty(w2.shape[0], dtype=np.int32)
    lib().orc_rowsum_i8(_p(w2), _p(out), w2.shape[0], w2.shape[1])
    return out


def _out_array(shape, out_mode):
    dt = {OUT_ACC_I32: np.int32, OUT_F32: np.float32, OUT_F16: np.uint16,
          OUT_REQUANT_I8: np.int8, OUT_FAKEQUANT_F32: np.float32}[out_mode]
    return np.empty(shape, dtype=dt)


def _bias_kind(bias):
    if bias is None:
        return BIAS_NONE, None
    if bias.dtype == np.float16:
        return BIAS_F16, np.ascontiguousarray(bias).view(np.uint16)
    return BIAS_F32, _f32(bias)


def qlinear(a, w, a_zp, a_scale, w_scale, bias=None, relu=False, out_mode=OUT_F32,
            out_scale=1.0, out_zp=0.0, out_qmin=0, out_qmax=255, out_offset=0, w_zp=None):
    """Integer-formulation quantized Linear.  ``a`` int8 [M,K] stored codes,
    ``a_zp`` the zero point of the stored codes, ``a_scale`` scalar or [M];
    ``w_zp`` int [N] zero points of the weight rows (None: symmetric weights)."""
    a = np.ascontiguousarray(a, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    M, K = a.shape
    N = w.shape[0]
    a_scale = _f32(a_scale).reshape(-1)
    per_row = int(a_scale.size != 1)
    assert a_scale.size in (1, M)
    w_scale = _f32(w_scale).reshape(-1)
    bk, b = _bias_kind(bias)
    out = _out_array((M, N), out_mode)
    if w_zp is not None:
        zw = np.ascontiguousarray(np.broadcast_to(np.asarray(w_zp, dtype=np.int32).reshape(-1), (N,)))
        lib().orc_qlinear_affine(_p(a), _p(w), _p(zw), M, N, K, int(a_zp), _p(a_scale), per_row,
                                 _p(w_scale), bk, _p(b), int(relu), out_mode, C.c_float(out_scale),
                                 C.c_float(out_zp), int(out_qmin), int(out_qmax), int(out_offset),
                                 _p(out))
        return out.view(np.float16) if out_mode == OUT_F16 else out
    lib().orc_qlinear(_p(a), _p(w), M, N, K, int(a_zp), _p(a_scale), per_row, _p(w_scale), bk,
                      _p(b), int(relu), out_mode, C.c_float(out_scale), C.c_float(out_zp),
                      int(out_qmin), int(out_qmax), int(out_offset), _p(out))
    return out.view(np.float16) if out_mode == OUT_F16 else out


def linear_faithful(x, wq, w_scale, w_zp, bias=None, relu=False, fq=None):
    """Lucid's float pass structure.  ``fq`` = (S, Z, qmin, qmax) or None."""
    x = _f32(x)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    M, K = x.shape
    N = wq.shape[0]
    out = np.empty((M, N), dtype=np.float32)
    S, Z, qmin, qmax = fq if fq is not None else (1.0, 0.0, 0, 255)
    b = None if bias is None else _f32(bias)
    lib().orc_linear_faithful(_p(x), _p(wq), _p(_f32(w_scale)), _p(_f32(w_zp)), _p(b), M, N, K,
                              int(relu), int(fq is not None), C.c_float(S), C.c_float(Z),
                              int(qmin), int(qmax), _p(out))
    return out


def conv_out_size(S, K, stride, pad_lo, pad_hi, dil):
    return lib().orc_conv_out_size(S, K, stride, pad_lo, pad_hi, dil)


def qconv2d(x, w, a_zp, a_scale, w_scale, stride=(1, 1), pad=(0, 0, 0, 0), dilation=(1, 1),
            groups=1, bias=None, relu=False, out_mode=OUT_F32, out_scale=1.0, out_zp=0.0,
            out_qmin=0, out_qmax=255, out_offset=0, w_zp=None):
    """Integer-formulation Conv2d.  ``x`` int8 NHWC codes, ``w`` int8
    [Cout,KH,KW,Cin/groups], ``pad`` = (h_lo, h_hi, w_lo, w_hi); ``w_zp`` int [Cout] zero
    points of the filters (None: symmetric).  Output NHWC."""
    x = np.ascontiguousarray(x, dtype=np.int8)
    w = np.ascontiguousarray(w, dtype=np.int8)
    B, H, W, Cin = x.shape
    Cout, KH, KW, Cg = w.shape
    assert Cg * groups == Cin
    OH = conv_out_size(H, KH, stride[0], pad[0], pad[1], dilation[0])
    OW = conv_out_size(W, KW, stride[1], pad[2], pad[3], dilation[1])
    bk, b = _bias_kind(bias)
    out = _out_array((B, OH, OW, Cout), out_mode)
    if w_zp is not None:
        zw = np.ascontiguousarray(np.broadcast_to(np.asarray(w_zp, dtype=np.int32).reshape(-1), (Cout,)))
        lib().orc_qconv2d_affine(_p(x), _p(w), _p(zw), B, H, W, Cin, Cout, KH, KW, stride[0],
                                 stride[1], pad[0], pad[1], pad[2], pad[3], dilation[0],
                                 dilation[1], groups, int(a_zp), C.c_float(a_scale),
                                 _p(_f32(w_scale)), bk, _p(b), int(relu), out_mode,
                                 C.c_float(out_scale), C.c_float(out_zp), int(out_qmin),
                                 int(out_qmax), int(out_offset), _p(out))
        return out.view(np.float16) if out_mode == OUT_F16 else out
    lib().orc_qconv2d(_p(x), _p(w), B, H, W, Cin, Cout, KH, KW, stride[0], stride[1], pad[0],
                      pad[1], pad[2], pad[3], dilation[0], dilation[1], groups, int(a_zp),
                      C.c_float(a_scale), _p(_f32(w_scale)), bk, _p(b), int(relu), out_mode,
                      C.c_float(out_scale), C.c_float(out_zp), int(out_qmin), int(out_qmax),
                      int(out_offset), _p(out))
    return out.view(np.float16) if out_mode == OUT_F16 else out


def conv2d_faithful(x, wq, w_scale, w_zp, bias=None, stride=(1, 1), pad=(0, 0), dilation=(1, 1),
                    groups=1, relu=False, fq=None):
    """Lucid's float pass structure.  NCHW input, OIHW int8 kernel."""
    x = _f32(x)
    wq = np.ascontiguousarray(wq, dtype=np.int8)
    B, Cin, H, W = x.shape
    Cout, _, KH, KW = wq.shape
    OH = conv_out_size(H, KH, stride[0], pad[0], pad[0], dilation[0])
    OW = conv_out_size(W, KW, stride[1], pad[1], pad[1], dilation[1])
    out = np.empty((B, Cout, OH, OW), dtype=np.float32)
    S, Z, qmin, qmax = fq if fq is not None else (1.0, 0.0, 0, 255)
    b = None if bias is None else _f32(bias)
    lib().orc_conv2d_faithful(_p(x), _p(wq), _p(_f32(w_scale)), _p(_f32(w_zp)), _p(b), B, Cin, H,
                              W, Cout, KH, KW, stride[0], stride[1], pad[0], pad[1], dilation[0],
                              dilation[1], groups, int(relu), int(fq is not None), C.c_float(S),
                              C.c_float(Z), int(qmin), int(qmax), _p(out))
    return out


def add_requant(qa, a_offset, sa, za, qb, b_offset, sb, zb, relu, S, Z, qmin, qmax, out_offset):
    qa = np.ascontiguousarray(qa, dtype=np.int8)
    qb = np.ascontiguousarray(qb, dtype=np.int8)
    out = np.empty(qa.shape, dtype=np.int8)
    lib().orc_add_requant(_p(qa), int(a_offset), C.c_float(sa), C.c_float(za), _p(qb),
                          int(b_offset), C.c_float(sb), C.c_float(zb), C.c_size_t(qa.size),
                          int(relu), C.c_float(S), C.c_float(Z), int(qmin), int(qmax),
                          int(out_offset), _p(out))
    return out


def maxpool2d_nhwc_i8(x, kernel, stride, pad):
    x = np.ascontiguousarray(x, dtype=np.int8)
    B, H, W, Cn = x.shape
    OH = (H + 2 * pad[0] - kernel[0]) // stride[0] + 1
    OW = (W + 2 * pad[1] - kernel[1]) // stride[1] + 1
    out = np.empty((B, OH, OW, Cn), dtype=np.int8)
    lib().orc_maxpool2d_nhwc_i8(_p(x), B, H, W, Cn, kernel[0], kernel[1], stride[0], stride[1],
                                pad[0], pad[1], _p(out))
    return out


def batchnorm_eval(x, mean, var, gamma=None, beta=None, eps=1e-5):
    """Eval-mode BatchNorm on ``(B, C, *)`` float32 with frozen statistics."""
    x = _f32(x)
    B, Cn = x.shape[0], x.shape[1]
    spatial = int(np.prod(x.shape[2:], dtype=np.int64))
    out = np.empty_like(x)
    g = None if gamma is None else _f32(gamma)
    b = None if beta is None else _f32(beta)
    lib().orc_batchnorm_eval(_p(x), _p(out), C.c_size_t(B), C.c_size_t(Cn), C.c_size_t(spatial),
                             _p(_f32(mean)), _p(_f32(var)), _p(g), _p(b), C.c_double(eps))
    return out
