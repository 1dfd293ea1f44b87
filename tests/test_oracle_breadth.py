"""The restatement of the module breadth (oracle/breadth.py) against what the mathematics
fixes: float64 closed forms of the activations, brute-force lookups, a scatter-form
transposed convolution against a direct sum, the LSTM against a float64 step."""

import numpy as np
import pytest

import oracle as O
import oracle.breadth as Br


def _table(rng, n=50, d=16):
    w = rng.standard_normal((n, d)).astype(np.float32)
    mn, mx = O.minmax(w, ch_axis=0)
    s, z = O.calc_qparams(mn, mx, True, -128, 127, True)
    return w, O.quantize(w, s, z, -128, 127, ch_axis=0), s, z


def test_embedding_is_a_row_gather_of_the_dequantized_table():
    rng = np.random.default_rng(0)
    w, q, s, z = _table(rng)
    idx = rng.integers(0, 50, (3, 7))
    out = Br.embedding(q, s, z, idx, padding_idx=4)
    assert out.shape == (3, 7, 16)
    for a in range(3):
        for b in range(7):
            i = idx[a, b]
            want = np.zeros(16, np.float32) if i == 4 else (q[i].astype(np.float32) - z[i]) * s[i]
            assert np.array_equal(out[a, b], want)
    # test_breadth.py:12-23: mean relative error of the int8 table under 2 %
    assert np.abs(out - np.where((idx == 4)[..., None], 0, w[idx])).mean() / np.abs(w[idx]).mean() < 0.02


@pytest.mark.parametrize("mode", ["sum", "mean", "max"])
def test_embedding_bag_pools_in_float64_agreement(mode):
    rng = np.random.default_rng(1)
    w, q, s, z = _table(rng)
    idx = np.array([1, 5, 9, 3, 7, 2, 8, 9, 9])
    off = np.array([0, 3, 5, 5])  # third bag empty, fourth runs to the end
    out = Br.embedding_bag(q, s, z, idx, off, mode, padding_idx=9)
    table = Br.dequantize_rows(q, s, z).astype(np.float64)
    bags = [[1, 5], [3, 7], [], [2, 8]]  # 9 is padding
    for b, members in enumerate(bags):
        if not members:
            want = np.zeros(16)
        elif mode == "sum":
            want = table[members].sum(0)
        elif mode == "mean":
            want = table[members].mean(0)
        else:
            want = table[members].max(0)
        assert np.allclose(out[b], want, rtol=1e-6, atol=1e-6)
    # 2-d indices: one bag per row
    out2 = Br.embedding_bag(q, s, z, np.array([[1, 5, 9], [3, 7, 2]]), None, mode, padding_idx=9)
    assert np.array_equal(out2[0], out[0])


def test_activation_formulas_against_float64():
    x = np.linspace(-9, 9, 20001).astype(np.float32)
    x64 = x.astype(np.float64)
    hs = np.clip((x64 + 3) / 6, 0, 1)
    want = {Br.SIGMOID: 1 / (1 + np.exp(-x64)), Br.HARDSWISH: x64 * hs, Br.HARDSIGMOID: hs,
            Br.TANH: np.tanh(x64), Br.ELU: np.where(x64 >= 0, x64, 0.7 * np.expm1(x64)),
            Br.LEAKY_RELU: np.where(x64 >= 0, x64, 0.2 * x64)}
    alpha = {Br.ELU: 0.7, Br.LEAKY_RELU: 0.2}
    for kind, ref in want.items():
        got = Br.act(kind, x, alpha.get(kind, 0.0))
        assert got.dtype == np.float32
        assert np.abs(got - ref).max() < 2e-6, kind
    # special values: the hard forms saturate, a NaN passes
    assert Br.act(Br.HARDSIGMOID, np.float32([-3, 3, -100, 100])).tolist() == [0, 1, 0, 1]
    assert np.isnan(Br.act(Br.HARDSWISH, np.float32([np.nan]))[0])
    assert Br.act(Br.SIGMOID, np.float32([0]))[0] == 0.5


def test_quantized_activation_on_codes_equals_the_float_formulation():
    rng = np.random.default_rng(2)
    s, z, S, Z = np.float32(0.05), np.float32(120), np.float32(1 / 255), np.float32(0)
    q = rng.integers(-128, 128, 4096).astype(np.int8)  # stored quint8 codes (code - 128)
    x = O.dequantize(q, s, z, code_offset=-128)
    for kind in range(6):
        codes = Br.quantized_act_codes(kind, q, -128, s, z, 0.3, S, Z, 0, 255, -128)
        floats = Br.quantized_act(kind, x, 0.3, S, Z, 0, 255)
        assert np.array_equal(O.dequantize(codes, S, Z, code_offset=-128), floats)


def test_lstm_against_a_float64_recurrence():
    rng = np.random.default_rng(3)
    T, B, I, H = 5, 3, 8, 6
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    wih, whh = (rng.standard_normal((4 * H, n)).astype(np.float32) * 0.3 for n in (I, H))
    bih, bhh = (rng.standard_normal(4 * H).astype(np.float32) * 0.1 for _ in range(2))
    h0, c0 = (rng.standard_normal((B, H)).astype(np.float32) for _ in range(2))
    y, hn, cn = Br.lstm(x, h0, c0, wih, whh, bih, bhh)
    h, c = h0.astype(np.float64), c0.astype(np.float64)
    sig = lambda v: 1 / (1 + np.exp(-v))
    for t in range(T):
        raw = x[t].astype(np.float64) @ wih.T + h @ whh.T + bih + bhh
        i, f, g, o = sig(raw[:, :H]), sig(raw[:, H:2 * H]), np.tanh(raw[:, 2 * H:3 * H]), sig(raw[:, 3 * H:])
        c = f * c + i * g
        h = o * np.tanh(c)
        assert np.allclose(y[t], h, atol=1e-5)
    assert np.allclose(hn, h, atol=1e-5) and np.allclose(cn, c, atol=1e-5)
    assert np.array_equal(y[-1], hn)


@pytest.mark.parametrize("proj", [0, 4])
@pytest.mark.parametrize("reverse", [False, True])
def test_lstm_projection_and_packed_schedule_against_torch(proj, reverse):
    """The oracle's projection (W_hr) and packed active-set schedule against torch.nn.LSTM fed a
    PackedSequence, and against running every sequence alone: a row's states must freeze at its
    own last step, in both directions."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(11 + proj + reverse)
    T, B, I, H = 6, 4, 5, 7
    R = proj if proj else H
    lengths = [6, 4, 4, 1]
    batch_sizes = [sum(1 for v in lengths if v > t) for t in range(T)]
    x = rng.standard_normal((T, B, I)).astype(np.float32)
    for b, n in enumerate(lengths):
        x[n:, b] = 0
    wih = (rng.standard_normal((4 * H, I)) * 0.3).astype(np.float32)
    whh = (rng.standard_normal((4 * H, R)) * 0.3).astype(np.float32)
    whr = (rng.standard_normal((proj, H)) * 0.3).astype(np.float32) if proj else None
    bih, bhh = ((rng.standard_normal(4 * H) * 0.1).astype(np.float32) for _ in range(2))
    h0 = rng.standard_normal((B, R)).astype(np.float32)
    c0 = rng.standard_normal((B, H)).astype(np.float32)
    y, hn, cn = Br.lstm(x, h0, c0, wih, whh, bih, bhh, w_hr=whr, batch_sizes=batch_sizes, reverse=reverse)
    # (1) every sequence on its own, dense
    for b, n in enumerate(lengths):
        xs = x[:n, b:b + 1]
        ys, hs, cs = Br.lstm(xs[::-1] if reverse else xs, h0[b:b + 1], c0[b:b + 1], wih, whh, bih, bhh, w_hr=whr)
        ys = ys[::-1] if reverse else ys
        # (numpy's matmul may round the last bit differently for a batch of one)
        assert np.allclose(y[:n, b], ys[:, 0], atol=1e-6) and not y[n:, b].any()
        assert np.allclose(hn[b], hs[0], atol=1e-6) and np.allclose(cn[b], cs[0], atol=1e-6)
    # (2) torch, the same weights, a packed batch (bidirectional: take the direction under test)
    m = torch.nn.LSTM(I, H, bidirectional=True, proj_size=proj)
    with torch.no_grad():
        for suffix in ("", "_reverse"):
            getattr(m, "weight_ih_l0" + suffix).copy_(torch.from_numpy(wih))
            getattr(m, "weight_hh_l0" + suffix).copy_(torch.from_numpy(whh))
            getattr(m, "bias_ih_l0" + suffix).copy_(torch.from_numpy(bih))
            getattr(m, "bias_hh_l0" + suffix).copy_(torch.from_numpy(bhh))
            if proj:
                getattr(m, "weight_hr_l0" + suffix).copy_(torch.from_numpy(whr))
        pk = torch.nn.utils.rnn.pack_padded_sequence(torch.from_numpy(x), lengths)
        h0t = torch.from_numpy(np.stack([h0, h0]))
        c0t = torch.from_numpy(np.stack([c0, c0]))
        out, (hT, cT) = m(pk, (h0t, c0t))
        out, _ = torch.nn.utils.rnn.pad_packed_sequence(out, total_length=T)
    d = 1 if reverse else 0
    assert np.allclose(y, out.numpy()[:, :, d * R:(d + 1) * R], atol=2e-6)
    assert np.allclose(hn, hT.numpy()[d], atol=2e-6) and np.allclose(cn, cT.numpy()[d], atol=2e-6)
    # a dense schedule is the plain recurrence
    yd, hd, cd = Br.lstm(x, h0, c0, wih, whh, bih, bhh, w_hr=whr, batch_sizes=[B] * T)
    y0, hh0, cc0 = Br.lstm(x, h0, c0, wih, whh, bih, bhh, w_hr=whr)
    assert np.array_equal(yd, y0) and np.array_equal(hd, hh0) and np.array_equal(cd, cc0)


@pytest.mark.parametrize("stride,padding,output_padding,dilation,groups",
                         [((2, 2), (1, 1), (1, 1), (1, 1), 1), ((1, 1), (0, 0), (0, 0), (1, 1), 1),
                          ((3, 2), (2, 0), (2, 1), (1, 1), 1), ((2, 2), (1, 1), (0, 0), (2, 1), 2)])
def test_conv_transpose_scatter_form_against_the_direct_sum(stride, padding, output_padding, dilation, groups):
    rng = np.random.default_rng(4)
    B, Cin, Cout, H, W, kh, kw = 2, 4, 6, 5, 4, 3, 2
    x = rng.standard_normal((B, Cin, H, W))
    w = rng.standard_normal((Cin, Cout // groups, kh, kw))
    bias = rng.standard_normal(Cout)
    out = Br.conv_transpose2d(x, w, bias, stride, padding, output_padding, dilation, groups)
    (sh, sw), (ph, pw), (dh, dw) = stride, padding, dilation
    OH = (H - 1) * sh - 2 * ph + dh * (kh - 1) + output_padding[0] + 1
    OW = (W - 1) * sw - 2 * pw + dw * (kw - 1) + output_padding[1] + 1
    assert out.shape == (B, Cout, OH, OW)
    cig, cog = Cin // groups, Cout // groups
    want = np.zeros_like(out)
    for b in range(B):
        for co in range(Cout):
            g = co // cog
            for oh in range(OH):
                for ow in range(OW):
                    acc = bias[co]
                    for ci in range(g * cig, (g + 1) * cig):
                        for i in range(kh):
                            for j in range(kw):
                                nh, nw = oh + ph - i * dh, ow + pw - j * dw
                                if nh % sh or nw % sw:
                                    continue
                                h, wd = nh // sh, nw // sw
                                if 0 <= h < H and 0 <= wd < W:
                                    acc += x[b, ci, h, wd] * w[ci, co - g * cog, i, j]
                    want[b, co, oh, ow] = acc
    assert np.allclose(out, want, atol=1e-10)


@pytest.mark.parametrize("stride,pad,dilation,groups", [
    ((1, 1, 1), ((0, 0),) * 3, (1, 1, 1), 1), ((2, 1, 2), ((1, 1), (0, 2), (1, 0)), (1, 1, 1), 1),
    ((1, 2, 1), ((1, 1),) * 3, (2, 1, 1), 2), ((1, 1, 1), ((2, 2), (1, 1), (0, 0)), (1, 2, 2), 4)])
def test_qconv3d_accumulation_against_scipy_correlate(stride, pad, dilation, groups):
    """The oracle's Conv3d (numpy tap gather + its qlinear per group) against an independent
    routine: scipy's N-d cross-correlation of the centred codes with the (zero-dilated) kernel,
    strided by slicing.  With unit scales and no bias the float32 output is the exact integer
    sum of (x - zp) * w, so the comparison is exact; a wrong tap order, a transposed kernel, a
    group mix-up or padding with anything but the zero point would show."""
    from scipy.signal import correlate
    rng = np.random.default_rng(11 + groups)
    B, C, Co, K3 = 2, 8, 12, (3, 2, 3)
    x = rng.integers(-128, 128, (B, C, 6, 7, 8)).astype(np.int8)
    w = rng.integers(-127, 128, (Co, C // groups, *K3)).astype(np.int8)
    zp = -37
    got = Br.qconv3d(x, w, zp, np.float32(1.0), np.ones(Co, np.float32), stride=stride, pad=pad, dilation=dilation,
                     groups=groups, out_mode=O.OUT_F32)
    xc = np.pad(x.astype(np.int64) - zp, ((0, 0), (0, 0), *pad))            # padding = zero point -> 0
    wd = np.zeros((Co, C // groups, *[d * (k - 1) + 1 for k, d in zip(K3, dilation)]), np.int64)
    wd[(slice(None), slice(None), *[slice(None, None, d) for d in dilation])] = w
    Cg, Og = C // groups, Co // groups
    want = np.zeros(got.shape, np.int64)
    for b in range(B):
        for o in range(Co):
            g = o // Og
            full = sum(correlate(xc[b, g * Cg + c], wd[o, c], mode="valid", method="direct") for c in range(Cg))
            want[b, o] = full[::stride[0], ::stride[1], ::stride[2]]
    assert got.shape == want.shape and np.array_equal(got.astype(np.int64), want)


@pytest.mark.parametrize("stride,padding,output_padding,dilation,groups", [
    ((1, 1, 1), (0, 0, 0), (0, 0, 0), (1, 1, 1), 1), ((2, 3, 2), (1, 0, 1), (1, 2, 0), (1, 1, 1), 1),
    ((2, 1, 2), (0, 1, 0), (0, 0, 1), (2, 1, 1), 2)])
def test_qconv_transpose3d_against_the_scatter_definition(stride, padding, output_padding, dilation, groups):
    """The oracle's ConvTranspose3d (zero insertion + flipped kernel + its Conv3d) against the
    definition: every input sample adds sample * kernel into the output at stride * position
    + dilation * tap - padding.  Unit scales, no bias: exact integers."""
    rng = np.random.default_rng(5 + groups)
    B, Cin, Cout, K3 = 2, 4, 6, (2, 3, 2)
    x = rng.integers(-128, 128, (B, Cin, 3, 4, 3)).astype(np.int8)
    w = rng.integers(-127, 128, (Cin, Cout // groups, *K3)).astype(np.int8)
    zp = 21
    got = Br.qconv_transpose3d(x, w, zp, np.float32(1.0), np.ones(Cout // groups, np.float32), stride=stride,
                               padding=padding, output_padding=output_padding, dilation=dilation, groups=groups,
                               out_mode=O.OUT_F32)
    size = [(n - 1) * s - 2 * p + d * (k - 1) + op + 1
            for n, s, p, d, k, op in zip(x.shape[2:], stride, padding, dilation, K3, output_padding)]
    full = np.zeros((B, Cout, *[n + 2 * p for n, p in zip(size, padding)]), np.int64)
    cig, cog = Cin // groups, Cout // groups
    xc = x.astype(np.int64) - zp
    for ci in range(Cin):
        g = ci // cig
        for idx in np.ndindex(*x.shape[2:]):
            for tap in np.ndindex(*K3):
                pos = tuple(i * s + t * d for i, s, t, d in zip(idx, stride, tap, dilation))
                full[(slice(None), slice(g * cog, (g + 1) * cog), *pos)] += \
                    xc[(slice(None), ci, *idx)][:, None] * w[(ci, slice(None), *tap)][None, :]
    want = full[(slice(None), slice(None), *[slice(p, p + n) for p, n in zip(padding, size)])]
    assert got.shape == want.shape and np.array_equal(got.astype(np.int64), want)


# ------------------------------------------------------------------ eval-mode BatchNorm
def test_batchnorm_eval_restates_the_reference_steps():
    """rstd through double, then g * (x - m) * r + b in float32 left to right
    (CpuBackend.h:9190-9198): pinned against the same steps in numpy float32, against torch's
    batch_norm within rounding, and on closed forms a dropped or swapped term would break."""
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    for shape in [(3, 5), (2, 4, 9), (2, 6, 7, 5), (2, 3, 4, 5, 6)]:
        Cn = shape[1]
        x = rng.standard_normal(shape).astype(np.float32) * 3
        m = rng.standard_normal(Cn).astype(np.float32)
        v = rng.uniform(0.1, 4.0, Cn).astype(np.float32)
        g = rng.uniform(0.5, 1.5, Cn).astype(np.float32)
        b = rng.standard_normal(Cn).astype(np.float32)
        y = O.batchnorm_eval(x, m, v, g, b, 1e-5)
        bc = (1, Cn) + (1,) * (len(shape) - 2)
        r = (np.float32(1.0) / np.sqrt(v.astype(np.float64) + 1e-5).astype(np.float32)).astype(np.float32)
        exp = ((g.reshape(bc) * (x - m.reshape(bc))).astype(np.float32) * r.reshape(bc)).astype(np.float32) \
            + b.reshape(bc)
        assert np.array_equal(y.view(np.uint32), exp.astype(np.float32).view(np.uint32))
        t = torch.nn.functional.batch_norm(torch.from_numpy(x), torch.from_numpy(m), torch.from_numpy(v),
                                           torch.from_numpy(g), torch.from_numpy(b), False, 0.0, 1e-5).numpy()
        assert np.allclose(y, t, rtol=2e-6, atol=2e-6)
        # no affine parameters = gamma 1, beta 0
        assert np.array_equal(O.batchnorm_eval(x, m, v, None, None, 1e-5),
                              O.batchnorm_eval(x, m, v, np.ones(Cn), np.zeros(Cn), 1e-5))
    # mean 0, var 1 - eps, gamma 1, beta 0: the identity; x == mean: exactly beta
    x = rng.standard_normal((2, 3, 8)).astype(np.float32)
    one_minus = np.full(3, 1.0 - 1e-5, np.float64).astype(np.float32)
    y = O.batchnorm_eval(x, np.zeros(3), one_minus, None, None, 1e-5)
    assert np.allclose(y, x, rtol=1e-6)
    y = O.batchnorm_eval(np.broadcast_to(np.float32([1, 2, 3])[None, :, None], (2, 3, 8)), [1, 2, 3], [4, 5, 6],
                         [7, 8, 9], [0.5, -0.5, 0.25], 1e-5)
    assert np.array_equal(y, np.broadcast_to(np.float32([0.5, -0.5, 0.25])[None, :, None], (2, 3, 8)))
