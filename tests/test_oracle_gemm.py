"""Pins the CPU oracle's integer GEMM, the quantized Linear / Conv2d integer
formulation, and the float ("faithful") restatement of Lucid's own pass
structure.

Independent truths used: numpy int64 matmul (exact), a pure-Python triple
loop on tiny shapes, algebraic invariants of exact integer arithmetic, and
torch.nn.functional.conv2d on integer-valued float64 tensors (exact).
"""

import numpy as np
import pytest

import oracle as O


def _codes(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


# ------------------------------------------------------------------ int32 accumulators
def test_igemm_tiny_brute_force():
    rng = np.random.default_rng(0)
    a, w = _codes(rng, (3, 5)), _codes(rng, (4, 5))
    expect = [[sum(int(a[m, k]) * int(w[n, k]) for k in range(5)) for n in range(4)]
              for m in range(3)]
    assert O.igemm(a, w).tolist() == expect


@pytest.mark.parametrize("M,N,K", [(1, 7, 64), (17, 33, 129), (64, 256, 784), (5, 10, 4096)])
def test_igemm_matches_numpy_int64(M, N, K):
    rng = np.random.default_rng(M * 1000 + N)
    a, w = _codes(rng, (M, K)), _codes(rng, (N, K))
    assert np.array_equal(O.igemm(a, w), a.astype(np.int64) @ w.astype(np.int64).T)


def test_igemm_extreme_codes_do_not_overflow():
    K = 4096
    a = np.full((2, K), -128, np.int8)
    w = np.full((3, K), -128, np.int8)
    assert (O.igemm(a, w) == 128 * 128 * K).all()
    w[:] = 127
    assert (O.igemm(a, w) == -128 * 127 * K).all()


def test_igemm_invariants():
    rng = np.random.default_rng(1)
    a, w = _codes(rng, (9, 200), -60, 60), _codes(rng, (11, 200))
    a2 = _codes(rng, (9, 200), -60, 60)
    acc = O.igemm(a, w)
    # K-split additivity
    assert np.array_equal(acc, O.igemm(a[:, :77], w[:, :77]) + O.igemm(a[:, 77:], w[:, 77:]))
    # linearity in the activation operand (kept inside int8)
    assert np.array_equal(O.igemm((a + a2).astype(np.int8), w), acc + O.igemm(a2, w))
    # row / column permutation
    pm, pn, pk = rng.permutation(9), rng.permutation(11), rng.permutation(200)
    assert np.array_equal(O.igemm(a[pm][:, pk], w[pn][:, pk]), acc[pm][:, pn])


def test_recentring_identity():
    # sum (xq - Z) w == sum (xq - 128) w - (Z - 128) sum w, with xq a quint8 code
    rng = np.random.default_rng(2)
    xq = rng.integers(0, 256, (13, 300)).astype(np.int16)
    w = _codes(rng, (21, 300))
    Z = 117
    true = O.igemm_a16((xq - Z).astype(np.int16), w)
    a8 = (xq - 128).astype(np.int8)
    acc = O.igemm(a8, w).astype(np.int64)
    assert np.array_equal(true, acc - (Z - 128) * O.rowsum_i8(w).astype(np.int64)[None, :])


# ------------------------------------------------------------------ Linear, integer formulation
def _linear_case(rng, M, N, K, per_row):
    x = rng.standard_normal((M, K)).astype(np.float32)
    wf = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.05).astype(np.float32)
    mn, mx = O.minmax(wf, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    wq = O.quantize(wf, ws, wz, -128, 127, ch_axis=0)
    if per_row:
        mn, mx = O.minmax(x, ch_axis=0)
        xs, xz = O.calc_qparams(mn, mx, True, -128, 127, True)
        xq = O.quantize(x, xs, xz, -128, 127, ch_axis=0)
        a_zp = 0
        xg = O.dequantize(xq, xs, xz, ch_axis=0)
    else:
        mn, mx = O.minmax(x)
        xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
        xq = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
        a_zp = int(xz[0]) - 128
        xg = O.fake_quantize(x, xs, xz, 0, 255)
    return dict(xq=xq, a_zp=a_zp, xs=xs, wq=wq, ws=ws, wz=wz, bias=bias, xg=xg)


@pytest.mark.parametrize("per_row", [False, True])
@pytest.mark.parametrize("M,N,K", [(64, 256, 784), (64, 10, 256), (16, 48, 512)])
def test_integer_linear_tracks_float_path(M, N, K, per_row):
    """The integer formulation is the algebraic identity of Lucid's float
    formulation; float outputs must agree within 1e-3 relative."""
    c = _linear_case(np.random.default_rng(M + N + K), M, N, K, per_row)
    y_int = O.qlinear(c["xq"], c["wq"], c["a_zp"], c["xs"], c["ws"], bias=c["bias"],
                      out_mode=O.OUT_F32)
    y_ref = O.linear_faithful(c["xg"], c["wq"], c["ws"], c["wz"], bias=c["bias"])
    scale = np.abs(y_ref).max()
    assert np.abs(y_int - y_ref).max() <= 1e-3 * scale
    # float64 evaluation of the same sum agrees even more tightly
    y64 = c["xg"].astype(np.float64) @ (c["wq"].astype(np.float64) * c["ws"][:, None]).T + c["bias"]
    assert np.abs(y_int - y64).max() <= 2e-5 * scale


def test_requant_codes_vs_float_path_are_within_one_lsb_near_ties():
    c = _linear_case(np.random.default_rng(5), 64, 256, 784, False)
    y_ref = O.linear_faithful(c["xg"], c["wq"], c["ws"], c["wz"], bias=c["bias"], relu=True)
    mn, mx = O.minmax(y_ref)
    S, Z = O.calc_qparams(mn, mx, False, 0, 255, False)
    codes_ref = O.quantize(y_ref, S, Z, 0, 255, q_dtype=O.I16)
    codes_int = O.qlinear(c["xq"], c["wq"], c["a_zp"], c["xs"], c["ws"], bias=c["bias"],
                          relu=True, out_mode=O.OUT_REQUANT_I8, out_scale=S[0], out_zp=Z[0],
                          out_offset=-128).astype(np.int16) + 128
    diff = codes_int - codes_ref
    assert np.abs(diff).max() <= 1
    bad = diff != 0
    assert bad.mean() < 2e-3
    t = y_ref[bad] / S[0]
    assert (np.abs(t - np.floor(t) - 0.5) < 1e-3).all()  # every mismatch sits on a tie


def test_epilogue_modes_compose_from_pinned_pieces():
    c = _linear_case(np.random.default_rng(6), 16, 48, 512, False)
    kw = dict(a_zp=c["a_zp"], a_scale=c["xs"], w_scale=c["ws"], bias=c["bias"], relu=True)
    y = O.qlinear(c["xq"], c["wq"], out_mode=O.OUT_F32, **kw)
    assert (y >= 0).all()
    S, Z = np.float32(0.013), np.float32(3.0)
    fq = O.qlinear(c["xq"], c["wq"], out_mode=O.OUT_FAKEQUANT_F32, out_scale=S, out_zp=Z, **kw)
    assert np.array_equal(fq, O.fake_quantize(y, S, Z, 0, 255))
    rq = O.qlinear(c["xq"], c["wq"], out_mode=O.OUT_REQUANT_I8, out_scale=S, out_zp=Z,
                   out_offset=-128, **kw)
    assert np.array_equal(rq, O.quantize(y, S, Z, 0, 255, code_offset=-128))
    h = O.qlinear(c["xq"], c["wq"], out_mode=O.OUT_F16, **kw)
    with np.errstate(over="ignore"):
        assert np.array_equal(h.view(np.uint16), y.astype(np.float16).view(np.uint16))
    acc = O.qlinear(c["xq"], c["wq"], out_mode=O.OUT_ACC_I32, **kw)
    assert np.array_equal(acc, O.igemm(c["xq"], c["wq"]))


def test_f16_bias_is_widened_before_the_add():
    rng = np.random.default_rng(8)
    a, w = _codes(rng, (4, 64)), _codes(rng, (6, 64))
    b16 = (rng.standard_normal(6) * 0.02).astype(np.float16)
    y16 = O.qlinear(a, w, 0, 0.01, np.full(6, 0.002, np.float32), bias=b16, out_mode=O.OUT_F32)
    y32 = O.qlinear(a, w, 0, 0.01, np.full(6, 0.002, np.float32), bias=b16.astype(np.float32),
                    out_mode=O.OUT_F32)
    assert np.array_equal(y16, y32)


# ------------------------------------------------------------------ convolution
def _np_conv_acc(x, w, stride, pad, dil, groups, pad_code):
    """Explicit gather + numpy int64 matmul.  x NHWC, w [Cout,KH,KW,Cg]."""
    B, H, W, Cin = x.shape
    Cout, KH, KW, Cg = w.shape
    xp = np.full((B, H + pad[0] + pad[1], W + pad[2] + pad[3], Cin), pad_code, np.int64)
    xp[:, pad[0]:pad[0] + H, pad[2]:pad[2] + W] = x
    OH = (H + pad[0] + pad[1] - dil[0] * (KH - 1) - 1) // stride[0] + 1
    OW = (W + pad[2] + pad[3] - dil[1] * (KW - 1) - 1) // stride[1] + 1
    out = np.zeros((B, OH, OW, Cout), np.int64)
    Og = Cout // groups
    for g in range(groups):
        for kh in range(KH):
            for kw in range(KW):
                patch = xp[:, kh * dil[0]: kh * dil[0] + (OH - 1) * stride[0] + 1: stride[0],
                           kw * dil[1]: kw * dil[1] + (OW - 1) * stride[1] + 1: stride[1],
                           g * Cg:(g + 1) * Cg]
                out[..., g * Og:(g + 1) * Og] += patch @ w[g * Og:(g + 1) * Og, kh, kw].astype(
                    np.int64).T
    return out


CONV_CASES = [
    # B,H,W,Cin,Cout,KH,KW,stride,pad(hlo,hhi,wlo,whi),dil,groups
    (2, 9, 11, 8, 12, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 1),
    (1, 14, 14, 3, 16, 7, 7, (2, 2), (3, 3, 3, 3), (1, 1), 1),
    (2, 8, 8, 16, 32, 1, 1, (1, 1), (0, 0, 0, 0), (1, 1), 1),
    (1, 10, 9, 8, 8, 3, 3, (2, 1), (0, 1, 1, 2), (1, 2), 2),
    (1, 6, 6, 4, 4, 3, 3, (1, 1), (1, 1, 1, 1), (1, 1), 4),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_qconv_accumulators_exact(case):
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups = case
    rng = np.random.default_rng(sum(case[:7]))
    x = _codes(rng, (B, H, W, Cin))
    w = _codes(rng, (Cout, KH, KW, Cin // groups))
    a_zp = -11
    acc = O.qconv2d(x, w, a_zp, 0.02, np.ones(Cout, np.float32), stride=st, pad=pad, dilation=dil,
                    groups=groups, out_mode=O.OUT_ACC_I32)
    assert np.array_equal(acc, _np_conv_acc(x, w, st, pad, dil, groups, a_zp))


@pytest.mark.parametrize("case", CONV_CASES[:3])
def test_qconv_matches_torch_exact_integer_conv(case):
    torch = pytest.importorskip("torch")
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups = case
    rng = np.random.default_rng(99)
    x = _codes(rng, (B, H, W, Cin))
    w = _codes(rng, (Cout, KH, KW, Cin // groups))
    a_zp = 5
    acc = O.qconv2d(x, w, a_zp, 0.02, np.ones(Cout, np.float32), stride=st, pad=pad, dilation=dil,
                    groups=groups, out_mode=O.OUT_ACC_I32)
    # (x - zp) conv w with true zero padding == acc - zp * sum(w)  (float64: exact)
    xt = torch.from_numpy((x.astype(np.float64) - a_zp).transpose(0, 3, 1, 2).copy())
    wt = torch.from_numpy(w.astype(np.float64).transpose(0, 3, 1, 2).copy())
    ref = torch.nn.functional.conv2d(xt, wt, None, st, (pad[0], pad[2]), dil, groups)
    ref = ref.numpy().transpose(0, 2, 3, 1)
    wsum = w.reshape(Cout, -1).astype(np.int64).sum(1)
    assert np.array_equal(acc.astype(np.int64) - a_zp * wsum, ref.astype(np.int64))


def test_conv_out_size_formula():
    # lucid/_C/nn/ConvNd.cpp:56-59
    assert O.conv_out_size(224, 7, 2, 3, 3, 1) == 112
    assert O.conv_out_size(56, 3, 1, 1, 1, 1) == 56
    assert O.conv_out_size(56, 3, 2, 1, 1, 1) == 28
    assert O.conv_out_size(10, 3, 1, 0, 0, 2) == 6


@pytest.mark.parametrize("case", CONV_CASES[:3] + CONV_CASES[4:])
def test_integer_conv_tracks_float_path(case):
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups = case
    rng = np.random.default_rng(17)
    x = rng.uniform(0, 1, (B, Cin, H, W)).astype(np.float32)
    wf = (rng.standard_normal((Cout, Cin // groups, KH, KW)) * 0.1).astype(np.float32)
    bias = (rng.standard_normal(Cout) * 0.1).astype(np.float32)
    mn, mx = O.minmax(wf, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    wq = O.quantize(wf, ws, wz, -128, 127, ch_axis=0)
    mn, mx = O.minmax(x)
    xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
    xg = O.fake_quantize(x, xs, xz, 0, 255)
    y_ref = O.conv2d_faithful(xg, wq, ws, wz, bias=bias, stride=st, pad=(pad[0], pad[2]),
                              dilation=dil, groups=groups, relu=True)
    xq = O.quantize(x.transpose(0, 2, 3, 1), xs, xz, 0, 255, code_offset=-128)
    y_int = O.qconv2d(xq, wq.transpose(0, 2, 3, 1), int(xz[0]) - 128, xs[0], ws, stride=st,
                      pad=pad, dilation=dil, groups=groups, bias=bias, relu=True,
                      out_mode=O.OUT_F32)
    assert np.abs(y_int.transpose(0, 3, 1, 2) - y_ref).max() <= 1e-3 * np.abs(y_ref).max()


def test_float_conv_matches_torch():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 6, 9, 8)).astype(np.float32)
    wq = _codes(rng, (8, 3, 3, 3))
    ws = rng.uniform(0.001, 0.01, 8).astype(np.float32)
    bias = rng.standard_normal(8).astype(np.float32)
    y = O.conv2d_faithful(x, wq, ws, np.zeros(8, np.float32), bias=bias, stride=(2, 1),
                          pad=(1, 1), groups=2)
    wf = torch.from_numpy(wq.astype(np.float32) * ws[:, None, None, None])
    ref = torch.nn.functional.conv2d(torch.from_numpy(x), wf, torch.from_numpy(bias), (2, 1),
                                     (1, 1), 1, 2)
    assert np.allclose(y, ref.numpy(), atol=1e-4)


# ------------------------------------------------------------------ residual join, pooling
def test_add_relu_requant_matches_float_composition():
    # nn/quantized/functional_module.py:228-230  fq(relu(x + y))
    rng = np.random.default_rng(4)
    qa, qb = _codes(rng, 5000), _codes(rng, 5000)
    sa, za, sb, zb = np.float32(0.021), 3.0, np.float32(0.034), 7.0
    xa = O.dequantize(qa, sa, za, code_offset=-128)
    xb = O.dequantize(qb, sb, zb, code_offset=-128)
    y = np.maximum(xa + xb, np.float32(0))
    S, Z = np.float32(0.05), 0.0
    expect = O.quantize(y, S, Z, 0, 255, code_offset=-128)
    got = O.add_requant(qa, -128, sa, za, qb, -128, sb, zb, True, S, Z, 0, 255, -128)
    assert np.array_equal(got, expect)


def test_maxpool_on_codes_commutes_with_quantize():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 9, 9, 4)).astype(np.float32)
    s, z = np.float32(0.03), 100.0
    q = O.quantize(x, s, z, 0, 255, code_offset=-128)
    pooled = O.maxpool2d_nhwc_i8(q, (3, 3), (2, 2), (1, 1))
    xt = torch.from_numpy(O.dequantize(q, s, z, code_offset=-128).transpose(0, 3, 1, 2).copy())
    ref = torch.nn.functional.max_pool2d(xt, 3, 2, 1).numpy().transpose(0, 2, 3, 1)
    assert np.array_equal(O.dequantize(pooled, s, z, code_offset=-128), ref)


# ------------------------------------------------------------------ affine weights
def _affine_weight_case(rng, N, K):
    """Per-channel affine int8 weight codes the way from_float makes them: min / max per row,
    affine qparams on [-128, 127], quantize."""
    wf = (rng.standard_normal((N, K)) * 0.1 + rng.uniform(-0.15, 0.15, (N, 1))).astype(np.float32)
    mn, mx = O.minmax(wf, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, False, -128, 127, True)
    wq = O.quantize(wf, ws, wz, -128, 127, ch_axis=0)
    return wf, wq, ws, wz


@pytest.mark.parametrize("M,N,K", [(5, 7, 3), (33, 20, 147), (16, 48, 512)])
def test_affine_weight_linear_is_the_exact_integer_sum(M, N, K):
    """Accumulator under the scales = sum_k (a - za) * (w - zw[n]), checked through the
    float32 output against an int64 numpy evaluation put through the same float steps, and
    through the correction identity that the GPU path uses."""
    rng = np.random.default_rng(M * N + K)
    a, w = _codes(rng, (M, K)), _codes(rng, (N, K))
    zw = rng.integers(-128, 128, N).astype(np.int32)
    za = -37
    a_scale = np.float32(0.0173)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    got = O.qlinear(a, w, za, a_scale, w_scale, bias=bias, out_mode=O.OUT_F32, w_zp=zw)
    eff = (a.astype(np.int64) - za) @ (w.astype(np.int64) - zw[:, None]).T
    exp = eff.astype(np.float32) * (a_scale * w_scale)[None, :] + bias[None, :]
    assert np.array_equal(got.view(np.uint32), exp.astype(np.float32).view(np.uint32))
    # acc - za*wsum - zw*asum + K*za*zw is the same integer
    acc = O.igemm(a, w).astype(np.int64)
    ident = (acc - za * w.astype(np.int64).sum(1)[None, :] - zw[None, :] * a.astype(np.int64).sum(1)[:, None]
             + K * za * zw[None, :].astype(np.int64))
    assert np.array_equal(ident, eff)
    # zero weight zero points: the symmetric function, bit for bit, in every output form
    for mode in (O.OUT_F32, O.OUT_F16, O.OUT_REQUANT_I8, O.OUT_FAKEQUANT_F32):
        kw = dict(bias=bias, relu=True, out_mode=mode, out_scale=0.05, out_zp=3.0, out_offset=-128)
        y0 = O.qlinear(a, w, za, a_scale, w_scale, **kw)
        y1 = O.qlinear(a, w, za, a_scale, w_scale, w_zp=np.zeros(N, np.int32), **kw)
        assert np.array_equal(y0.view(np.uint8), y1.view(np.uint8))


def test_affine_weight_linear_special_cases():
    rng = np.random.default_rng(8)
    M, N, K = 9, 6, 40
    a = _codes(rng, (M, K))
    zw = np.array([-128, -5, 0, 17, 127, 64], np.int32)
    # every code equal to its row's zero point = an all-zero float weight: output == bias
    w = np.repeat(zw.astype(np.int8)[:, None], K, axis=1)
    bias = rng.standard_normal(N).astype(np.float32)
    y = O.qlinear(a, w, 11, 0.02, np.full(N, 0.003, np.float32), bias=bias, w_zp=zw)
    assert np.array_equal(y, np.broadcast_to(bias, (M, N)))
    # every activation code equal to its zero point = an all-zero input: output == bias
    w = _codes(rng, (N, K))
    y = O.qlinear(np.full((M, K), 11, np.int8), w, 11, 0.02, np.full(N, 0.003, np.float32), bias=bias, w_zp=zw)
    assert np.array_equal(y, np.broadcast_to(bias, (M, N)))
    # raw accumulators ignore both zero points
    assert np.array_equal(O.qlinear(a, w, 11, 1.0, np.ones(N, np.float32), out_mode=O.OUT_ACC_I32, w_zp=zw),
                          O.igemm(a, w))


def test_affine_weight_linear_tracks_lucids_float_path():
    """Against the float restatement of Lucid's composite (dequantize the affine weight, float
    GEMM, lucid/nn/quantized/linear.py:199-215), which takes the weight zero points itself."""
    rng = np.random.default_rng(21)
    M, N, K = 32, 40, 256
    wf, wq, ws, wz = _affine_weight_case(rng, N, K)
    assert np.any(wz != 0)
    x = rng.uniform(-1, 2, (M, K)).astype(np.float32)
    mn, mx = O.minmax(x)
    xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
    xq = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
    xg = O.fake_quantize(x, xs, xz, 0, 255)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    y_int = O.qlinear(xq, wq, int(xz[0]) - 128, xs, ws, bias=bias, w_zp=wz.astype(np.int32))
    y_ref = O.linear_faithful(xg, wq, ws, wz, bias=bias)
    assert np.abs(y_int - y_ref).max() <= 1e-3 * np.abs(y_ref).max()
    # and ignoring the zero points is visibly wrong, so the check above has teeth
    y_sym = O.qlinear(xq, wq, int(xz[0]) - 128, xs, ws, bias=bias)
    assert np.abs(y_sym - y_ref).max() > 0.05 * np.abs(y_ref).max()


@pytest.mark.parametrize("case", CONV_CASES)
def test_affine_weight_conv_is_the_exact_integer_sum(case):
    B, H, W, Cin, Cout, KH, KW, st, pad, dil, groups = case
    rng = np.random.default_rng(5 + sum(case[:7]))
    x = _codes(rng, (B, H, W, Cin))
    w = _codes(rng, (Cout, KH, KW, Cin // groups))
    zw = rng.integers(-128, 128, Cout).astype(np.int32)
    za = 23
    a_scale = np.float32(0.021)
    w_scale = rng.uniform(0.0005, 0.004, Cout).astype(np.float32)
    bias = rng.standard_normal(Cout).astype(np.float32)
    got = O.qconv2d(x, w, za, a_scale, w_scale, stride=st, pad=pad, dilation=dil, groups=groups,
                    bias=bias, out_mode=O.OUT_F32, w_zp=zw)
    # (x - za) conv (w - zw) with true zero padding, by the numpy accumulator on shifted operands
    eff = _np_conv_acc(x.astype(np.int64) - za, w.astype(np.int64) - zw[:, None, None, None], st, pad, dil,
                       groups, 0)
    exp = eff.astype(np.float32) * (a_scale * w_scale) + bias
    assert np.array_equal(got.view(np.uint32), exp.astype(np.float32).view(np.uint32))
    y0 = O.qconv2d(x, w, za, a_scale, w_scale, stride=st, pad=pad, dilation=dil, groups=groups, bias=bias)
    y1 = O.qconv2d(x, w, za, a_scale, w_scale, stride=st, pad=pad, dilation=dil, groups=groups, bias=bias,
                   w_zp=np.zeros(Cout, np.int32))
    assert np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
