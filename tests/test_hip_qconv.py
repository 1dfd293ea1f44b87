"""GPU parity of the quantized Conv2d forward (``lq_qconv2d_i8``) and its
layout helpers against the CPU oracle: int32 accumulators and requantized
codes bit for bit on every route (1x1-as-GEMM, implicit GEMM, explicit im2col,
naive), including ResNet-50's layer shapes, asymmetric padding, dilation,
groups and ragged extents."""

import numpy as np
import pytest

import lucid_amd as L
from lucid_amd import _C, _ops
import oracle as O

pytestmark = pytest.mark.gpu

GEMM, IMPLICIT, IM2COL, NAIVE = _ops.CONV_GEMM, _ops.CONV_IMPLICIT, _ops.CONV_IM2COL, _ops.CONV_NAIVE


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


def codes(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


CASES = [
    # B, H, W, Cin, Cout, KH, KW, stride, pad(hlo,hhi,wlo,whi), dil, groups, routes
    (2, 9, 11, 16, 24, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, (IMPLICIT, IM2COL, NAIVE)),
    (1, 14, 14, 3, 16, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1), 1, (IM2COL, NAIVE)),       # stem-like
    (2, 8, 8, 32, 64, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 1, (GEMM, IMPLICIT, IM2COL, NAIVE)),
    (2, 8, 8, 64, 32, 1, 1, (2, 2), (0, 0, 0, 0), (1, 1), 1, (IMPLICIT, NAIVE)),       # downsample
    (1, 10, 9, 32, 16, 3, 3, (2, 1), (0, 1, 1, 2), (1, 2), 2, (IMPLICIT, IM2COL, NAIVE)),
    (1, 6, 6, 8, 8, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 4, (IM2COL, NAIVE)),
    (3, 17, 13, 48, 70, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, (IMPLICIT, NAIVE)),     # ragged M, N
    (2, 28, 28, 128, 128, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, (IMPLICIT,)),          # ResNet 3x3
    (2, 14, 14, 256, 256, 3, 3, (2, 2), (1, 1, 1, 1), (1, 1), 1, (IMPLICIT,)),          # stride-2 3x3
    (2, 14, 14, 1024, 256, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 1, (GEMM,)),
    (2, 56, 56, 64, 64, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1, (IMPLICIT,)),            # N = 64 tile
]


@pytest.mark.parametrize("case", CASES)
def test_accumulators_exact_on_every_route(case):
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups, routes = case
    rng = np.random.default_rng(sum(case[:7]))
    x = codes(rng, (B, H, W, Cin))
    w = codes(rng, (Cout, KH, KW, Cin // groups))
    a_zp = -17
    exp = O.qconv2d(x, w, a_zp, 1.0, np.ones(Cout, np.float32), stride=st, pad=pad, dilation=dil,
                    groups=groups, out_mode=O.OUT_ACC_I32)
    xd, wd = hip(x), hip(w)
    for route in routes:
        got = _ops.qconv2d_i8(xd, wd, a_zp=a_zp, stride=st, pad=pad, dilation=dil, groups=groups,
                              out_mode=_ops.OUT_ACC_I32, path=route).numpy()
        assert got.shape == exp.shape and np.array_equal(got, exp), f"route {route}"
    auto = _ops.qconv2d_i8(xd, wd, a_zp=a_zp, stride=st, pad=pad, dilation=dil, groups=groups,
                           out_mode=_ops.OUT_ACC_I32).numpy()
    assert np.array_equal(auto, exp)


@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[3], CASES[4], CASES[7]])
@pytest.mark.parametrize("relu,bias_kind", [(True, "f32"), (False, "f32"), (True, None)])
def test_epilogue_bit_exact(case, relu, bias_kind):
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups, routes = case
    rng = np.random.default_rng(7 + sum(case[:7]))
    x = codes(rng, (B, H, W, Cin))
    w = codes(rng, (Cout, KH, KW, Cin // groups))
    a_zp = int(rng.integers(-128, -60))
    a_scale = np.float32(rng.uniform(0.005, 0.03))
    w_scale = rng.uniform(0.0005, 0.004, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32) if bias_kind else None
    kw = dict(stride=st, pad=pad, dilation=dil, groups=groups, bias=bias, relu=relu)
    y = O.qconv2d(x, w, a_zp, a_scale, w_scale, out_mode=O.OUT_F32, **kw)
    S = np.float32(np.abs(y).max() / 200 + 1e-6)
    Z = np.float32(0.0 if relu else 128.0)
    wsum = _ops.rowsum_i8(hip(w))
    assert np.array_equal(wsum.numpy(), O.rowsum_i8(w))
    dkw = dict(stride=st, pad=pad, dilation=dil, groups=groups, relu=relu, a_zp=a_zp,
               a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum,
               bias=None if bias is None else hip(bias), out_scale=hip(S), out_zp=hip(Z),
               out_qmin=0, out_qmax=255, out_offset=-128)
    for route in routes:
        for mode in (_ops.OUT_F32, _ops.OUT_REQUANT_I8, _ops.OUT_FAKEQUANT_F32):
            got = _ops.qconv2d_i8(hip(x), hip(w), out_mode=mode, path=route, **dkw).numpy()
            exp = O.qconv2d(x, w, a_zp, a_scale, w_scale, out_mode=mode, out_scale=S, out_zp=Z,
                            out_qmin=0, out_qmax=255, out_offset=-128, **kw)
            if mode == _ops.OUT_REQUANT_I8:
                assert np.array_equal(got, exp), (route, mode)
            else:
                assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), (route, mode)


def test_layout_helpers_round_trip():
    rng = np.random.default_rng(3)
    B, Cc, H, W = 2, 37, 9, 11
    x = (rng.standard_normal((B, Cc, H, W)) * 2).astype(np.float32)
    s, z = hip(np.float32(0.03)), hip(np.float32(120.0))
    q = L.Tensor.empty((B, H, W, Cc), L.int8, "hip")
    _C.call("lq_quantize_nchw_to_nhwc", hip(x).data_ptr, q.data_ptr, -128, B, Cc, H, W,
            s.data_ptr, z.data_ptr, 0, 255, None)
    exp_q = O.quantize(x.transpose(0, 2, 3, 1), 0.03, 120.0, 0, 255, code_offset=-128)
    assert np.array_equal(q.numpy(), exp_q)
    out = L.Tensor.empty((B, Cc, H, W), L.float32, "hip")
    _C.call("lq_dequantize_nhwc_to_nchw", q.data_ptr, -128, out.data_ptr, B, Cc, H, W, s.data_ptr,
            z.data_ptr, None)
    exp = O.dequantize(exp_q, 0.03, 120.0, code_offset=-128).transpose(0, 3, 1, 2)
    assert np.array_equal(out.numpy().view(np.uint32), np.ascontiguousarray(exp).view(np.uint32))
    assert np.array_equal(out.numpy().view(np.uint32),
                          O.fake_quantize(x, 0.03, 120.0, 0, 255).view(np.uint32))
    w = codes(rng, (10, 6, 3, 5))
    wo = L.Tensor.empty((10, 3, 5, 6), L.int8, "hip")
    _C.call("lq_repack_oihw_to_ohwi_i8", hip(w).data_ptr, wo.data_ptr, 10, 6, 3, 5, None)
    assert np.array_equal(wo.numpy(), w.transpose(0, 2, 3, 1))


@pytest.mark.parametrize("C", [70, 64, 48])          # scalar kernel; 16-channel lanes
@pytest.mark.parametrize("k,s,p", [((3, 3), (2, 2), (1, 1)), ((2, 2), (2, 2), (0, 0)), ((2, 2), (1, 2), (1, 1)),
                                   ((3, 3), (1, 1), (0, 1)), ((3, 2), (2, 1), (1, 0)), ((5, 5), (3, 3), (2, 2))])
def test_maxpool_on_codes(C, k, s, p):
    """Windows with compile-time sizes (3 x 3, 2 x 2: every tap requested up front) and the general
    loop, with and without padding: the oracle's maxima, code for code."""
    rng = np.random.default_rng(4 + C + k[0])
    B, H, W = 2, 13, 12
    x = codes(rng, (B, H, W, C))
    OH, OW = (H + 2 * p[0] - k[0]) // s[0] + 1, (W + 2 * p[1] - k[1]) // s[1] + 1
    out = L.Tensor.empty((B, OH, OW, C), L.int8, "hip")
    _C.call("lq_maxpool2d_nhwc_i8", hip(x).data_ptr, out.data_ptr, B, H, W, C, k[0], k[1], s[0], s[1], p[0], p[1], None)
    assert np.array_equal(out.numpy(), O.maxpool2d_nhwc_i8(x, k, s, p))


def test_argument_validation():
    x, w = hip(np.zeros((1, 4, 4, 16), np.int8)), hip(np.zeros((8, 3, 3, 16), np.int8))
    with pytest.raises(L.ShapeMismatch):
        _ops.qconv2d_i8(x, hip(np.zeros((8, 3, 3, 8), np.int8)), a_zp=0, out_mode=0)
    with pytest.raises(L.ShapeMismatch):        # kernel larger than the padded image
        _ops.qconv2d_i8(hip(np.zeros((1, 2, 2, 16), np.int8)), w, a_zp=0, out_mode=0)
    with pytest.raises(ValueError):             # implicit route needs Cin/groups % 16 == 0
        _ops.qconv2d_i8(hip(np.zeros((1, 4, 4, 8), np.int8)), hip(np.zeros((8, 3, 3, 8), np.int8)),
                        a_zp=0, out_mode=0, path=IMPLICIT, pad=(1, 1, 1, 1))
    with pytest.raises(ValueError):             # zero point without the filter sums
        _ops.qconv2d_i8(x, w, a_zp=3, a_scale=hip(np.float32(1)), w_scale=hip(np.ones(8, np.float32)),
                        pad=(1, 1, 1, 1))


_NP_MODE = {1: "reflect", 2: "edge", 3: "wrap"}


@pytest.mark.parametrize("mode", [1, 2, 3])
@pytest.mark.parametrize("shape,pad", [((2, 9, 11, 16), (1, 1, 1, 1)), ((1, 5, 7, 3), (2, 0, 1, 3)),
                                        ((3, 8, 8, 64), (3, 3, 3, 3)), ((1, 4, 4, 20), (0, 0, 0, 0))])
def test_padding_modes_on_codes(mode, shape, pad):
    """F.pad reflect / replicate / circular gathers the image; on a tensor that lies
    on a grid the codes are gathered the same way (torch's F.pad semantics are
    numpy's reflect / edge / wrap)."""
    rng = np.random.default_rng(sum(shape) + mode)
    x = codes(rng, shape)
    B, H, W, Cc = shape
    out = L.Tensor.empty((B, H + pad[0] + pad[1], W + pad[2] + pad[3], Cc), L.int8, "hip")
    _C.call("lq_pad_nhwc_i8", hip(x).data_ptr, out.data_ptr, B, H, W, Cc, *pad, mode, None)
    exp = np.pad(x, ((0, 0), (pad[0], pad[1]), (pad[2], pad[3]), (0, 0)), mode=_NP_MODE[mode])
    assert np.array_equal(out.numpy(), exp)
    import torch

    tmode = {1: "reflect", 2: "replicate", 3: "circular"}[mode]
    t = torch.nn.functional.pad(torch.from_numpy(x.astype(np.float32)).permute(0, 3, 1, 2),
                                (pad[2], pad[3], pad[0], pad[1]), mode=tmode)
    assert np.array_equal(t.permute(0, 2, 3, 1).numpy().astype(np.int8), exp)


@pytest.mark.parametrize("padding_mode", ["reflect", "replicate", "circular"])
def test_conv_module_with_a_padding_mode(padding_mode):
    """nnq.Conv2d with padding_mode != zeros: pre-pad, then convolve with padding 0
    (lucid/nn/modules/conv.py:104-123)."""
    import lucid_amd.nn.quantized as nnq
    import lucid_amd.quantization as Q
    from lucid_amd._tensor import Grid, Tensor

    rng = np.random.default_rng(5)
    B, H, W, Cin, Cout = 2, 9, 10, 16, 24
    x = rng.integers(0, 256, (B, H, W, Cin)).astype(np.int16)
    wq = codes(rng, (Cout, Cin, 3, 3), -127, 127)
    ws = rng.uniform(0.001, 0.01, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    conv = nnq.Conv2d(Cin, Cout, 3, padding=1)
    conv.padding_mode = padding_mode
    state = {"weight_int8": wq, "weight_scale": ws, "weight_zero_point": np.zeros(Cout, np.float32),
             "bias": bias, "scale": np.float32(0.05), "zero_point": np.float32(120.0)}
    conv.load_state_dict({k: L.tensor(v, device="hip") for k, v in state.items()})
    in_scale, in_zp = np.float32(0.02), 128
    grid = Grid(hip((x - 128).astype(np.int8)), L.tensor(np.float32(in_scale), device="hip"),
                L.tensor(np.float32(in_zp), device="hip"), Q.quint8, -128, in_zp, "nhwc")
    y = conv(Tensor.on_grid((B, Cin, H, W), grid))
    got = y._grid.codes.numpy()
    xp = np.pad((x - 128).astype(np.int8), ((0, 0), (1, 1), (1, 1), (0, 0)),
                mode={"reflect": "reflect", "replicate": "edge", "circular": "wrap"}[padding_mode])
    exp = O.qconv2d(xp, np.ascontiguousarray(wq.transpose(0, 2, 3, 1)), in_zp - 128, in_scale, ws, bias=bias,
                    out_mode=O.OUT_REQUANT_I8, out_scale=0.05, out_zp=120.0, out_qmin=0, out_qmax=255,
                    out_offset=-128)
    assert np.array_equal(got, exp)


@pytest.mark.parametrize("shape,path", [((2, 14, 14, 64, 256, 1, 1), 0), ((2, 14, 14, 64, 96, 3, 3), 0),
                                        ((3, 9, 7, 32, 40, 3, 3), 0), ((2, 9, 7, 6, 10, 3, 3), 0),
                                        ((2, 9, 7, 32, 40, 3, 3), 4)])
def test_fused_join_equals_conv_then_add_requant(shape, path):
    """The residual add on codes fused into the epilogue gives the bits of the two-kernel
    form: conv -> stored codes -> lq_add_requant_i8 (functional_module.py:224-230)."""
    from lucid_amd import _C, _ops
    B, H, W, Cin, Cout, KH, KW = shape
    rng = np.random.default_rng(sum(shape))
    x = rng.integers(-128, 128, (B, H, W, Cin)).astype(np.int8)
    w = rng.integers(-127, 128, (Cout, KH, KW, Cin)).astype(np.int8)
    ws = (rng.random(Cout).astype(np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(Cout).astype(np.float32) * 0.1
    hip = lambda a: L.tensor(a, device="hip")
    dw, dx = hip(w), hip(x)
    common = dict(a_zp=-3, a_scale=hip(np.float32(0.02)), w_scale=hip(ws), wsum=_ops.rowsum_i8(dw),
                  bias=hip(bias), pad=(1, 1, 1, 1) if KH == 3 else (0, 0, 0, 0), relu=False,
                  out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(0.03)), out_zp=hip(np.float32(120.0)),
                  out_qmin=0, out_qmax=255, out_offset=-128, path=path)
    first = _ops.qconv2d_i8(dx, dw, **common)
    other = rng.integers(-128, 128, first.shape).astype(np.int8)
    d_other = hip(other)
    s2, z2 = hip(np.float32(0.025)), hip(np.float32(131.0))
    S, Z = hip(np.float32(0.04)), hip(np.float32(7.0))
    for relu in (True, False):
        want = L.Tensor.empty(first.shape, L.int8, "hip")
        _C.call("lq_add_requant_i8", first.data_ptr, -128, common["out_scale"].data_ptr, common["out_zp"].data_ptr,
                d_other.data_ptr, -128, s2.data_ptr, z2.data_ptr, first.numel, int(relu), S.data_ptr, Z.data_ptr,
                0, 255, -128, want.data_ptr, None)
        fused = _ops.qconv2d_i8(dx, dw, **common, join=dict(q=d_other, offset=-128, scale=s2, zp=z2, relu=relu,
                                                             out_scale=S, out_zp=Z, out_qmin=0, out_qmax=255,
                                                             out_offset=-128))
        assert np.array_equal(fused.numpy(), want.numpy())
    # the oracle's two steps, once
    o1 = O.qconv2d(x, w, -3, 0.02, ws, pad=common["pad"], bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=0.03,
                   out_zp=120.0, out_qmin=0, out_qmax=255, out_offset=-128)
    o2 = O.add_requant(o1, -128, 0.03, 120.0, other, -128, 0.025, 131.0, False, 0.04, 7.0, 0, 255, -128)
    assert np.array_equal(fused.numpy(), o2)


def test_join_needs_the_requantizing_mode():
    from lucid_amd import _ops
    hip = lambda a: L.tensor(a, device="hip")
    x, w = hip(np.zeros((1, 4, 4, 16), np.int8)), hip(np.zeros((16, 1, 1, 16), np.int8))
    one = hip(np.float32(1.0))
    j = dict(q=hip(np.zeros((1, 4, 4, 16), np.int8)), offset=0, scale=one, zp=one, relu=False, out_scale=one,
             out_zp=one, out_qmin=-128, out_qmax=127, out_offset=0)
    with pytest.raises(ValueError, match="REQUANT_I8"):
        _ops.qconv2d_i8(x, w, a_zp=0, a_scale=one, w_scale=hip(np.ones(16, np.float32)), out_mode=_ops.OUT_F32,
                        join=j)


@pytest.mark.parametrize("B,H,W,Cin,Cout,KH,KW,stride,pad", [
    (2, 224, 224, 3, 64, 7, 7, (2, 2), (3, 3, 3, 3)),   # the ResNet stem
    (3, 17, 13, 3, 24, 3, 3, (1, 1), (1, 1, 1, 1)),
    (2, 20, 9, 1, 16, 5, 2, (2, 1), (2, 1, 0, 1)),      # one channel, asymmetric padding, odd sizes
    (2, 11, 11, 4, 40, 3, 5, (1, 3), (0, 0, 2, 2)),
])
def test_packed_route_for_few_input_channels(B, H, W, Cin, Cout, KH, KW, stride, pad):
    """At most four input channels: the packed 4-channel gather gives the accumulators and codes of
    the oracle (and so of the im2col route it replaces)."""
    from lucid_amd import _ops
    rng = np.random.default_rng(B + H + Cout)
    x = rng.integers(-128, 128, (B, H, W, Cin)).astype(np.int8)
    w = rng.integers(-127, 128, (Cout, KH, KW, Cin)).astype(np.int8)
    ws = (rng.random(Cout).astype(np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(Cout).astype(np.float32) * 0.1
    hip = lambda a: L.tensor(a, device="hip")
    dx, dw = hip(x), hip(w)
    acc = _ops.qconv2d_i8(dx, dw, a_zp=0, stride=stride, pad=pad, out_mode=_ops.OUT_ACC_I32, path=_ops.CONV_PACKED4)
    assert np.array_equal(acc.numpy(), O.qconv2d(x, w, 0, 1.0, np.ones(Cout, np.float32), stride=stride, pad=pad,
                                                 out_mode=O.OUT_ACC_I32))
    kw = dict(a_zp=-7, a_scale=hip(np.float32(0.02)), w_scale=hip(ws), wsum=_ops.rowsum_i8(dw), bias=hip(bias),
              stride=stride, pad=pad, relu=True, out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(0.05)),
              out_zp=hip(np.float32(0.0)), out_qmin=0, out_qmax=255, out_offset=-128)
    auto = _ops.qconv2d_i8(dx, dw, **kw)                       # chooses the packed route
    want = O.qconv2d(x, w, -7, 0.02, ws, stride=stride, pad=pad, bias=bias, relu=True, out_mode=O.OUT_REQUANT_I8,
                     out_scale=0.05, out_zp=0.0, out_qmin=0, out_qmax=255, out_offset=-128)
    assert np.array_equal(auto.numpy(), want)
    assert np.array_equal(_ops.qconv2d_i8(dx, dw, **kw, path=_ops.CONV_IM2COL).numpy(), want)


@pytest.mark.parametrize("B,H,W,Cin,Cout,KH,KW,stride,pad", [
    (2, 224, 224, 3, 64, 7, 7, (2, 2), (3, 3, 3, 3)),   # the ResNet stem
    (3, 17, 13, 3, 24, 3, 3, (1, 1), (1, 1, 1, 1)),
    (2, 20, 9, 1, 16, 5, 2, (2, 1), (2, 1, 0, 1)),
    (2, 11, 11, 4, 40, 3, 5, (1, 3), (0, 0, 2, 2)),
])
def test_float_image_quantized_into_the_packed_form(B, H, W, Cin, Cout, KH, KW, stride, pad):
    """A float NCHW image quantized straight into the packed four-channel image, convolved with the
    filter packed once: the codes of the oracle's quantize followed by its convolution, and the
    packed image itself holds the oracle's codes inside and the zero-point code everywhere else."""
    rng = np.random.default_rng(7 * B + H + Cout)
    x = (rng.standard_normal((B, Cin, H, W)) * 1.3).astype(np.float32)
    x.reshape(-1)[:6] = [np.nan, np.inf, -np.inf, 1e30, -1e30, 0.0125]
    w = rng.integers(-127, 128, (Cout, KH, KW, Cin)).astype(np.int8)
    ws = (rng.random(Cout).astype(np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(Cout).astype(np.float32) * 0.1
    s_in, z_in = np.float32(0.025), np.float32(119.0)
    xq = np.ascontiguousarray(O.quantize(x, s_in, z_in, 0, 255, code_offset=-128).transpose(0, 2, 3, 1))
    a_zp = 119 - 128
    Hp, Wp, KWp = _ops.packed4_geometry(H, W, Cin, KW, stride[1], pad)
    assert KWp == (KW + 3) // 4 * 4 and Hp == H + pad[0] + pad[1] and Wp % 4 == 0
    OW = O.conv_out_size(W, KW, stride[1], pad[2], pad[3], 1)
    assert Wp >= max(W + pad[2] + pad[3], (OW - 1) * stride[1] + KWp)
    image = _ops.quantize_nchw_to_packed4(hip(x), hip(s_in), hip(z_in), 0, 255, -128, a_zp, pad, Hp, Wp)
    want_image = np.full((B, Hp, Wp, 4), a_zp, np.int8)
    want_image[:, pad[0]:pad[0] + H, pad[2]:pad[2] + W, :Cin] = xq
    assert np.array_equal(image.numpy(), want_image)
    dw = hip(w)
    wp = _ops.pack4_filter_i8(dw)
    want_w = np.zeros((Cout, KH, KWp, 4), np.int8)
    want_w[:, :, :KW, :Cin] = w
    assert np.array_equal(wp.numpy(), want_w)
    kw = dict(a_zp=a_zp, a_scale=hip(s_in), w_scale=hip(ws), wsum=_ops.rowsum_i8(dw), bias=hip(bias),
              stride=stride, pad=pad, relu=True, out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(0.05)),
              out_zp=hip(np.float32(3.0)), out_qmin=0, out_qmax=255, out_offset=-128)
    got = _ops.qconv2d_i8(image, wp, **kw, path=_ops.CONV_PREPACKED4, logical=(H, W, Cin, KW))
    want = O.qconv2d(xq, w, a_zp, s_in, ws, stride=stride, pad=pad, bias=bias, relu=True, out_mode=O.OUT_REQUANT_I8,
                     out_scale=0.05, out_zp=3.0, out_qmin=0, out_qmax=255, out_offset=-128)
    assert np.array_equal(got.numpy(), want)
    assert np.array_equal(_ops.qconv2d_i8(hip(xq), dw, **kw).numpy(), want)


@pytest.mark.parametrize("B,H,W,Cin,Cout,KH,KW,stride,pad,dil_h", [
    (2, 224, 224, 3, 64, 7, 7, (2, 2), (3, 3, 3, 3), 1),    # the ResNet stem: whole 16-byte stores
    (3, 17, 13, 3, 24, 3, 3, (1, 1), (1, 1, 1, 1), 1),      # one k step, a partial column tile
    (2, 20, 9, 1, 16, 5, 2, (2, 1), (2, 1, 0, 1), 2),       # dilated rows, one channel
    (2, 11, 11, 4, 40, 3, 5, (1, 3), (0, 0, 2, 2), 1),      # stride 3 along the row
    (1, 40, 37, 3, 160, 5, 5, (1, 2), (2, 2, 2, 2), 1),     # three column tiles, the last one partial
    (5, 33, 70, 2, 128, 8, 8, (3, 1), (1, 2, 3, 4), 1),     # K = 256, boxes past the right edge
])
def test_few_channel_kernel_with_the_filter_in_registers(B, H, W, Cin, Cout, KH, KW, stride, pad, dil_h):
    """tile_config 20 on the packed route: accumulators and every output form equal the oracle's."""
    rng = np.random.default_rng(11 * B + H + Cout)
    x = rng.integers(-128, 128, (B, H, W, Cin)).astype(np.int8)
    w = rng.integers(-127, 128, (Cout, KH, KW, Cin)).astype(np.int8)
    ws = (rng.random(Cout).astype(np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(Cout).astype(np.float32) * 0.1
    dx, dw = hip(x), hip(w)
    geo = dict(stride=stride, pad=pad, dilation=(dil_h, 1))
    acc = _ops.qconv2d_i8(dx, dw, a_zp=0, **geo, out_mode=_ops.OUT_ACC_I32, path=_ops.CONV_PACKED4, tile_config=20)
    assert _C.load().lq_last_tile_config() & 0xff == 20
    assert np.array_equal(acc.numpy(), O.qconv2d(x, w, 0, 1.0, np.ones(Cout, np.float32), **geo, out_mode=O.OUT_ACC_I32))
    common = dict(a_zp=-7, a_scale=hip(np.float32(0.02)), w_scale=hip(ws), wsum=_ops.rowsum_i8(dw), bias=hip(bias), **geo,
                  relu=True, path=_ops.CONV_PACKED4, tile_config=20)
    ocommon = dict(**geo, bias=bias, relu=True)
    for mode, omode in ((_ops.OUT_F32, O.OUT_F32), (_ops.OUT_F16, O.OUT_F16)):
        got = _ops.qconv2d_i8(dx, dw, **common, out_mode=mode).numpy()
        assert np.array_equal(got, O.qconv2d(x, w, -7, 0.02, ws, **ocommon, out_mode=omode))
    for mode, omode, okw in ((_ops.OUT_REQUANT_I8, O.OUT_REQUANT_I8, dict(out_offset=-128)),
                             (_ops.OUT_FAKEQUANT_F32, O.OUT_FAKEQUANT_F32, {})):
        got = _ops.qconv2d_i8(dx, dw, **common, out_mode=mode, out_scale=hip(np.float32(0.05)),
                              out_zp=hip(np.float32(3.0)), out_qmin=0, out_qmax=255, **okw).numpy()
        want = O.qconv2d(x, w, -7, 0.02, ws, **ocommon, out_mode=omode, out_scale=0.05, out_zp=3.0, out_qmin=0,
                         out_qmax=255, **okw)
        assert np.array_equal(got, want)
    # a signed output grid: the codes are not packed through the unsigned-byte conversion
    got = _ops.qconv2d_i8(dx, dw, **common, out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(0.05)),
                          out_zp=hip(np.float32(-20.0)), out_qmin=-128, out_qmax=127).numpy()
    assert np.array_equal(got, O.qconv2d(x, w, -7, 0.02, ws, **ocommon, out_mode=O.OUT_REQUANT_I8, out_scale=0.05,
                                         out_zp=-20.0, out_qmin=-128, out_qmax=127))


def test_few_channel_kernel_declines_long_filter_rows():
    x, w = hip(np.zeros((1, 20, 20, 3), np.int8)), hip(np.zeros((16, 11, 11, 3), np.int8))
    with pytest.raises(NotImplementedError, match="K <= 256"):          # 11 x 12 x 4 = 528 bytes
        _ops.qconv2d_i8(x, w, a_zp=0, out_mode=_ops.OUT_ACC_I32, path=_ops.CONV_PACKED4, tile_config=20)
    x16, w16 = hip(np.zeros((1, 8, 8, 16), np.int8)), hip(np.zeros((16, 3, 3, 16), np.int8))
    with pytest.raises(NotImplementedError, match="packed four-channel image"):
        _ops.qconv2d_i8(x16, w16, a_zp=0, out_mode=_ops.OUT_ACC_I32, tile_config=20)


@pytest.mark.parametrize("cin,relu,wzp,padding", [(3, True, 0, 3), (1, False, 0, "same"), (4, True, 0, 0),
                                                  (8, False, 0, 1), (3, False, 5, 1)])
def test_conv_module_taking_the_quantize_module(cin, relu, wzp, padding):
    """``conv(x, quantize=q)`` holds the codes of ``conv(q(x))``: through the packed image where the
    layer has at most four channels and symmetric filters, through ``q`` itself otherwise."""
    import lucid_amd.nn.quantized as nnq
    import lucid_amd.quantization as Q

    rng = np.random.default_rng(60 + cin)
    B, H, W, Cout, k = 2, 19, 23, 24, 5
    x = hip((rng.standard_normal((B, cin, H, W)) * 1.5).astype(np.float32))
    conv = (nnq.ConvReLU2d if relu else nnq.Conv2d)(cin, Cout, k, stride=1 if padding == "same" else 2, padding=padding)
    state = {"weight_int8": codes(rng, (Cout, cin, k, k), -127, 127),
             "weight_scale": rng.uniform(0.001, 0.01, Cout).astype(np.float32),
             "weight_zero_point": np.full(Cout, wzp, np.float32), "bias": rng.standard_normal(Cout).astype(np.float32),
             "scale": np.float32(0.05), "zero_point": np.float32(17.0)}
    conv.load_state_dict({k_: L.tensor(v, device="hip") for k_, v in state.items()})
    q = nnq.Quantize(hip(np.float32(0.03)), hip(np.float32(121.0)), Q.quint8)
    fused = conv(x, quantize=q)
    two = conv(q(x))
    assert fused.shape == two.shape and fused._grid.layout == two._grid.layout == "nhwc"
    assert np.array_equal(fused._grid.codes.numpy(), two._grid.codes.numpy())
    assert ("_w_packed4" in conv.__dict__) == (cin <= 4 and wzp == 0)
    # new weights drop the packed filter
    conv.load_state_dict({"weight_int8": L.tensor(-state["weight_int8"], device="hip")}, strict=False)
    assert conv.__dict__.get("_w_packed4") is None
    assert np.array_equal(conv(x, quantize=q)._grid.codes.numpy(), conv(q(x))._grid.codes.numpy())


def test_packed_operands_are_checked():
    one = hip(np.float32(1.0))
    image, wp = hip(np.zeros((1, 8, 12, 4), np.int8)), hip(np.zeros((16, 3, 4, 4), np.int8))
    kw = dict(a_zp=0, a_scale=one, w_scale=hip(np.ones(16, np.float32)), pad=(1, 1, 1, 1), path=_ops.CONV_PREPACKED4)
    with pytest.raises(ValueError, match="logical"):
        _ops.qconv2d_i8(image, wp, **kw)
    with pytest.raises(_C.ShapeMismatch, match="packed"):
        _ops.qconv2d_i8(image, wp, **kw, logical=(7, 7, 3, 3))        # the image of a 6 x 6 layer
    assert _ops.qconv2d_i8(image, wp, **kw, logical=(6, 6, 3, 3)).shape == (1, 6, 6, 16)
    with pytest.raises(ValueError, match="affine filters"):
        _ops.qconv2d_i8(image, wp, **kw, logical=(6, 6, 3, 3), wsum=hip(np.zeros(16, np.int32)),
                        w_zp=hip(np.ones(16, np.int32)))
    with pytest.raises(ValueError, match="Cin <= 4"):
        _ops.packed4_geometry(8, 8, 5, 3, 1, (0, 0, 0, 0))


# ------------------------------------------------------------------ affine filter codes
@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[2], CASES[4], CASES[5], CASES[6], CASES[8]])
def test_affine_filter_zero_points_on_every_route(case):
    """Per-channel affine filters (a zero point per output channel): every route and output
    form equals the oracle's term-by-term sum of (x - za) * (w - zw[co]) over the window, with
    taps in the padding contributing nothing, bit for bit."""
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups, routes = case
    rng = np.random.default_rng(31 + sum(case[:7]))
    x = codes(rng, (B, H, W, Cin))
    w = codes(rng, (Cout, KH, KW, Cin // groups))
    zw = rng.integers(-128, 128, Cout).astype(np.int32)
    zw[::5] = 0
    a_zp = int(rng.integers(-128, 128))
    a_scale = np.float32(rng.uniform(0.005, 0.03))
    w_scale = rng.uniform(0.0005, 0.004, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    kw = dict(stride=st, pad=pad, dilation=dil, groups=groups, bias=bias, relu=True)
    y = O.qconv2d(x, w, a_zp, a_scale, w_scale, w_zp=zw, **kw)
    S, Z = np.float32(y.max() / 250 + 1e-6), np.float32(1.0)
    xd, wd = hip(x), hip(w)
    dkw = dict(stride=st, pad=pad, dilation=dil, groups=groups, relu=True, a_zp=a_zp, a_scale=hip(a_scale),
               w_scale=hip(w_scale), wsum=_ops.rowsum_i8(wd), bias=hip(bias), out_scale=hip(S), out_zp=hip(Z),
               out_qmin=0, out_qmax=255, out_offset=-128, w_zp=hip(zw))
    for route in routes + (0,):
        for mode in (_ops.OUT_F32, _ops.OUT_REQUANT_I8):
            got = _ops.qconv2d_i8(xd, wd, out_mode=mode, path=route, **dkw).numpy()
            exp = O.qconv2d(x, w, a_zp, a_scale, w_scale, out_mode=mode, out_scale=S, out_zp=Z, out_qmin=0,
                            out_qmax=255, out_offset=-128, w_zp=zw, **kw)
            assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), (route, mode)
    sym = _ops.qconv2d_i8(xd, wd, out_mode=_ops.OUT_F32, **{**dkw, "w_zp": None}).numpy()
    assert not np.array_equal(sym, O.qconv2d(x, w, a_zp, a_scale, w_scale, w_zp=zw, **kw))


def test_affine_filters_with_the_fused_join():
    B, H, W, Cin, Cout = 2, 10, 10, 32, 48
    rng = np.random.default_rng(12)
    x, w = codes(rng, (B, H, W, Cin)), codes(rng, (Cout, 3, 3, Cin))
    zw = rng.integers(-90, 90, Cout).astype(np.int32)
    other = codes(rng, (B, H, W, Cout))
    a_scale, w_scale = np.float32(0.02), rng.uniform(0.0005, 0.004, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    xd, wd = hip(x), hip(w)
    join = dict(q=hip(other), offset=-128, scale=hip(np.float32(0.04)), zp=hip(np.float32(131.0)), relu=True,
                out_scale=hip(np.float32(0.06)), out_zp=hip(np.float32(0.0)), out_qmin=0, out_qmax=255,
                out_offset=-128)
    got = _ops.qconv2d_i8(xd, wd, a_zp=-3, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=_ops.rowsum_i8(wd),
                          bias=hip(bias), pad=(1, 1, 1, 1), out_mode=_ops.OUT_REQUANT_I8,
                          out_scale=hip(np.float32(0.05)), out_zp=hip(np.float32(120.0)), out_qmin=0,
                          out_qmax=255, out_offset=-128, join=join, w_zp=hip(zw)).numpy()
    c1 = O.qconv2d(x, w, -3, a_scale, w_scale, pad=(1, 1, 1, 1), bias=bias, out_mode=O.OUT_REQUANT_I8,
                   out_scale=0.05, out_zp=120.0, out_offset=-128, w_zp=zw)
    exp = O.add_requant(c1, -128, 0.05, 120.0, other, -128, 0.04, 131.0, True, 0.06, 0.0, 0, 255, -128)
    assert np.array_equal(got, exp)


@pytest.mark.parametrize("groups", [1, 2])
def test_conv_module_with_affine_filters(groups):
    """nnq.Conv2d and nnq.ConvTranspose2d loaded with non-zero weight zero points apply them:
    bit-exact against the oracle on the equivalent convolution."""
    import lucid_amd.nn.quantized as nnq
    import lucid_amd.quantization as Q
    from lucid_amd._tensor import Grid, Tensor

    rng = np.random.default_rng(50 + groups)
    B, H, W, Cin, Cout = 2, 9, 10, 16, 24
    x = rng.integers(0, 256, (B, H, W, Cin)).astype(np.int16)
    in_scale, in_zp = np.float32(0.02), 131
    grid = Grid(hip((x - 128).astype(np.int8)), L.tensor(np.float32(in_scale), device="hip"),
                L.tensor(np.float32(in_zp), device="hip"), Q.quint8, -128, in_zp, "nhwc")
    xin = Tensor.on_grid((B, Cin, H, W), grid)

    wq = codes(rng, (Cout, Cin // groups, 3, 3))
    ws = rng.uniform(0.001, 0.01, Cout).astype(np.float32)
    wz = rng.integers(-100, 100, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    conv = nnq.Conv2d(Cin, Cout, 3, padding=1, groups=groups)
    state = {"weight_int8": wq, "weight_scale": ws, "weight_zero_point": wz, "bias": bias,
             "scale": np.float32(0.05), "zero_point": np.float32(120.0)}
    conv.load_state_dict({k: L.tensor(v, device="hip") for k, v in state.items()})
    got = conv(xin)._grid.codes.numpy()
    exp = O.qconv2d((x - 128).astype(np.int8), np.ascontiguousarray(wq.transpose(0, 2, 3, 1)), in_zp - 128, in_scale,
                    ws, pad=(1, 1, 1, 1), groups=groups, bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=0.05,
                    out_zp=120.0, out_qmin=0, out_qmax=255, out_offset=-128, w_zp=wz.astype(np.int32))
    assert np.array_equal(got, exp)

    # transposed: weight (Cin, Cout/groups, kh, kw), qparams per output channel within a group
    og = Cout // groups
    wt = codes(rng, (Cin, og, 3, 3))
    wst = rng.uniform(0.001, 0.01, og).astype(np.float32)
    wzt = rng.integers(-100, 100, og).astype(np.float32)
    dec = nnq.ConvTranspose2d(Cin, Cout, 3, stride=2, padding=1, output_padding=1, groups=groups)
    state = {"weight_int8": wt, "weight_scale": wst, "weight_zero_point": wzt, "bias": bias,
             "scale": np.float32(0.05), "zero_point": np.float32(120.0)}
    dec.load_state_dict({k: L.tensor(v, device="hip") for k, v in state.items()})
    got = dec(xin)._grid.codes.numpy()
    # the equivalent convolution: zero-point codes between the samples, flipped kernel, channels
    # swapped inside each group, stride 1, padding k - 1 - p (+ output_padding at the high end)
    spread = np.full((B, 2 * H - 1, 2 * W - 1, Cin), in_zp - 128, np.int8)
    spread[:, ::2, ::2] = (x - 128).astype(np.int8)
    cig = Cin // groups
    weq = np.concatenate([np.transpose(wt[g * cig:(g + 1) * cig, :, ::-1, ::-1], (1, 2, 3, 0))
                          for g in range(groups)], axis=0)
    exp = O.qconv2d(spread, np.ascontiguousarray(weq), in_zp - 128, in_scale, np.tile(wst, groups),
                    pad=(1, 2, 1, 2), groups=groups, bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=0.05,
                    out_zp=120.0, out_qmin=0, out_qmax=255, out_offset=-128,
                    w_zp=np.tile(wzt, groups).astype(np.int32))
    assert np.array_equal(got, exp)


HALO_CASES = [
    # B, H, W, Cin, Cout, KH, KW, pad(hlo,hhi,wlo,whi), dil, groups
    (2, 28, 28, 128, 128, 3, 3, (1, 1, 1, 1), (1, 1), 1),     # ResNet 3x3, two 64-channel slices
    (2, 56, 56, 64, 64, 3, 3, (1, 1, 1, 1), (1, 1), 1),
    (3, 17, 13, 64, 70, 3, 3, (1, 1, 1, 1), (1, 1), 1),       # ragged box, ragged columns
    (1, 9, 20, 128, 48, 3, 2, (0, 2, 1, 0), (2, 3), 2),       # one-sided pads, dilation, groups
    (2, 7, 7, 192, 256, 5, 5, (2, 2, 2, 2), (1, 1), 1),       # image smaller than a box
    (1, 40, 6, 64, 33, 1, 3, (0, 0, 1, 1), (1, 1), 1),        # width below eight
]


@pytest.mark.parametrize("cfg", [15, 18, 19])
@pytest.mark.parametrize("case", HALO_CASES)
def test_halo_kernel_exact(case, cfg):
    """tile_config 15 / 18 / 19 - the stride-1 convolution that keeps the input halo of a box of
    256 / 128 / 64 outputs in LDS - against the oracle: accumulators, and the requantize / float32 /
    float16 / fake-quantize epilogues."""
    B, H, W, Cin, Cout, KH, KW, pad, dil, groups = case
    rng = np.random.default_rng(sum(case[:7]) + 15)
    x = codes(rng, (B, H, W, Cin))
    w = codes(rng, (Cout, KH, KW, Cin // groups))
    a_zp = int(rng.integers(-100, 100))
    geo = dict(stride=(1, 1), pad=pad, dilation=dil, groups=groups)
    xd, wd = hip(x), hip(w)
    exp = O.qconv2d(x, w, a_zp, 1.0, np.ones(Cout, np.float32), out_mode=O.OUT_ACC_I32, **geo)
    got = _ops.qconv2d_i8(xd, wd, a_zp=a_zp, out_mode=_ops.OUT_ACC_I32, path=IMPLICIT, tile_config=cfg, **geo).numpy()
    assert got.shape == exp.shape and np.array_equal(got, exp)
    a_scale = np.float32(0.02)
    w_scale = rng.uniform(0.0005, 0.004, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    y = O.qconv2d(x, w, a_zp, a_scale, w_scale, bias=bias, out_mode=O.OUT_F32, **geo)
    S, Z = np.float32(np.abs(y).max() / 200 + 1e-6), np.float32(0.0)
    dkw = dict(a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=_ops.rowsum_i8(wd), bias=hip(bias),
               relu=True, out_scale=hip(S), out_zp=hip(Z), out_qmin=0, out_qmax=255, out_offset=-128,
               path=IMPLICIT, tile_config=cfg, **geo)
    for mode in (_ops.OUT_REQUANT_I8, _ops.OUT_F32, _ops.OUT_F16, _ops.OUT_FAKEQUANT_F32):
        got = _ops.qconv2d_i8(xd, wd, out_mode=mode, **dkw).numpy()
        exp = O.qconv2d(x, w, a_zp, a_scale, w_scale, bias=bias, relu=True, out_mode=mode, out_scale=S, out_zp=Z,
                        out_qmin=0, out_qmax=255, out_offset=-128, **geo)
        if mode in (_ops.OUT_REQUANT_I8,):
            assert np.array_equal(got, exp), mode
        elif mode == _ops.OUT_F16:
            assert np.array_equal(got.view(np.uint16), exp.view(np.uint16)), mode
        else:
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32)), mode


def test_halo_kernel_refuses_what_it_is_not_built_for():
    rng = np.random.default_rng(3)
    x, w = hip(codes(rng, (1, 8, 8, 64))), hip(codes(rng, (64, 3, 3, 64)))
    with pytest.raises(NotImplementedError, match="stride 1"):
        _ops.qconv2d_i8(x, w, a_zp=0, stride=(2, 2), pad=(1, 1, 1, 1), out_mode=_ops.OUT_ACC_I32, path=IMPLICIT,
                        tile_config=15)
    x32, w32 = hip(codes(rng, (1, 8, 8, 32))), hip(codes(rng, (64, 3, 3, 32)))
    with pytest.raises(NotImplementedError, match="64 == 0"):
        _ops.qconv2d_i8(x32, w32, a_zp=0, pad=(1, 1, 1, 1), out_mode=_ops.OUT_ACC_I32, path=IMPLICIT, tile_config=15)


def _loaded(conv, wq, ws, bias, S, Z):
    state = {"weight_int8": wq, "weight_scale": ws, "weight_zero_point": np.zeros(len(ws), np.float32), "bias": bias,
             "scale": np.float32(S), "zero_point": np.float32(Z)}
    conv.load_state_dict({k: L.tensor(v, device="hip") for k, v in state.items()})
    return conv


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("geom", [dict(k=3, stride=1, padding=1, dilation=1, groups=1),
                                  dict(k=3, stride=2, padding=1, dilation=1, groups=2),
                                  dict(k=(1, 3), stride=1, padding=(0, 2), dilation=(1, 2), groups=1),
                                  dict(k=3, stride=2, padding="same", dilation=1, groups=1),
                                  dict(k=5, stride=1, padding="valid", dilation=1, groups=1)])
def test_float_input_form_of_quantized_conv2d(geom, relu):
    """nnq.Conv2d / ConvReLU2d on a plain float tensor take Lucid's float formulation
    (lucid/nn/quantized/conv.py:168-184): dequantized weight -> float32 convolution -> bias ->
    [ReLU] -> fake_quantize.  Against the oracle's pass-for-pass restatement: the float32 sums run
    in another order, so the tolerance is the reference's own (one quantization step where a value
    sits on a rounding tie, equal elsewhere)."""
    import lucid_amd.nn.quantized.intrinsic as nniq
    import lucid_amd.nn.quantized as nnq

    rng = np.random.default_rng(11)
    B, Cin, Cout, H, W = 2, 8, 12, 11, 13
    k = geom["k"] if isinstance(geom["k"], tuple) else (geom["k"], geom["k"])
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    wq = codes(rng, (Cout, Cin // geom["groups"], *k), -127, 127)
    ws = rng.uniform(0.002, 0.01, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    S, Z = 0.04, 128.0
    cls = nniq.ConvReLU2d if relu else nnq.Conv2d
    conv = _loaded(cls(Cin, Cout, k, stride=geom["stride"], padding=geom["padding"], dilation=geom["dilation"],
                       groups=geom["groups"]), wq, ws, bias, S, Z)
    y = conv(hip(x))
    assert y._grid is not None and y.shape[:2] == (B, Cout)
    got = y.numpy()
    pad = geom["padding"]
    xin = x
    if pad == "same":   # uneven amounts: the odd unit on the high side (lucid/nn/modules/conv.py:44-55)
        st = geom["stride"]
        amounts = []
        for n, kk in ((H, k[0]), (W, k[1])):
            out = (n + st - 1) // st
            tot = max(0, (out - 1) * st + kk - n)
            amounts.append((tot // 2, tot - tot // 2))
        xin = np.pad(x, ((0, 0), (0, 0), amounts[0], amounts[1]))
        pad = (0, 0)
    elif pad == "valid":
        pad = (0, 0)
    elif isinstance(pad, int):
        pad = (pad, pad)
    dil = geom["dilation"] if isinstance(geom["dilation"], tuple) else (geom["dilation"],) * 2
    exp = O.conv2d_faithful(xin, wq, ws, np.zeros(Cout, np.float32), bias=bias, stride=(geom["stride"],) * 2, pad=pad,
                            dilation=dil, groups=geom["groups"], relu=relu, fq=(S, Z, 0, 255))
    assert got.shape == exp.shape
    diff = np.abs(got - exp)
    assert diff.max() <= S * 1.0001
    assert np.mean(diff > 0) < 0.01


@pytest.mark.parametrize("padding_mode", ["reflect", "replicate", "circular"])
def test_float_input_form_with_a_padding_mode(padding_mode):
    """The float-input form pre-pads the float image as the float layer does; checked against the
    same layer fed the pre-padded image with padding 0."""
    import lucid_amd.nn.quantized as nnq

    rng = np.random.default_rng(12)
    B, Cin, Cout, H, W = 2, 4, 6, 9, 10
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    wq = codes(rng, (Cout, Cin, 3, 3), -127, 127)
    ws = rng.uniform(0.002, 0.01, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    conv = _loaded(nnq.Conv2d(Cin, Cout, 3, padding=(1, 2)), wq, ws, bias, 0.05, 100.0)
    conv.padding_mode = padding_mode
    got = conv(hip(x)).numpy()
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (2, 2)), mode={"reflect": "reflect", "replicate": "edge", "circular": "wrap"}[padding_mode])
    plain = _loaded(nnq.Conv2d(Cin, Cout, 3, padding=0), wq, ws, bias, 0.05, 100.0)
    want = plain(hip(xp)).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_float_input_form_of_quantized_conv1d_and_conv3d():
    """Conv1d / Conv3d on plain floats: within one output step of the same layer fed the input
    quantized on a fine grid (the int8 route), which the oracle pins bit for bit elsewhere."""
    import lucid_amd.nn.quantized as nnq

    rng = np.random.default_rng(13)
    S = 0.05
    # 1-d
    B, Cin, Cout, Ln = 2, 16, 8, 33
    x = (rng.integers(-100, 100, (B, Cin, Ln)) * 0.01).astype(np.float32)     # exactly on a 0.01 grid
    wq = codes(rng, (Cout, Cin, 3), -127, 127)
    ws = rng.uniform(0.002, 0.01, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    c1 = _loaded(nnq.Conv1d(Cin, Cout, 3, stride=2, padding=1), wq, ws, bias, S, 128.0)
    got = c1(hip(x)).numpy()
    xq = nnq.Quantize(L.tensor(np.float32(0.01), device="hip"), L.tensor(np.float32(128.0), device="hip"))(hip(x))
    want = c1(xq).numpy()
    assert got.shape == want.shape == (B, Cout, 17)
    assert np.abs(got - want).max() <= S * 1.0001 and np.mean(got != want) < 0.02
    # 3-d
    B, Cin, Cout, D, H, W = 1, 16, 8, 5, 6, 7
    x = (rng.integers(-100, 100, (B, Cin, D, H, W)) * 0.01).astype(np.float32)
    wq = codes(rng, (Cout, Cin, 3, 3, 3), -127, 127)
    c3 = _loaded(nnq.Conv3d(Cin, Cout, 3, padding=1), wq, ws, bias, S, 128.0)
    got = c3(hip(x)).numpy()
    want = c3(xq.__class__.on_grid(x.shape, nnq.Quantize(L.tensor(np.float32(0.01), device="hip"),
                                                         L.tensor(np.float32(128.0), device="hip"))(hip(x))._grid)).numpy()
    assert got.shape == want.shape == (B, Cout, D, H, W)
    assert np.abs(got - want).max() <= S * 1.0001 and np.mean(got != want) < 0.02
