"""Quantized module breadth on the device against the restatement (oracle/breadth.py)
and the reference's own tests (lucid/test/unit/quantization/test_breadth.py,
test_module_breadth.py)."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.nn.quantized as nnq
import lucid_amd.quantization as Q
import oracle as O
import oracle.breadth as Br

pytestmark = pytest.mark.gpu


def hip(a, dtype=None):
    return L.tensor(a, device="hip") if dtype is None else L.tensor(np.asarray(a, dtype), device="hip")


def volume_codes(t):
    """Stored codes of a 5-d activation in (B, C, D, H, W) order, whichever layout it is kept in."""
    codes = t._grid.codes.numpy()
    return np.ascontiguousarray(np.moveaxis(codes, -1, 1)) if t._grid.layout == "nhwc" else codes


# ---------------------------------------------------------------- embeddings
@pytest.mark.parametrize("num,dim,idx_dtype", [(100, 32, np.int64), (257, 30, np.int32), (5000, 768, np.int64)])
def test_embedding_bit_exact(num, dim, idx_dtype):
    emb = nn.Embedding(num, dim, padding_idx=3)
    q = nnq.Embedding.from_float(emb)
    assert q.weight_int8.dtype is L.int8 and q.weight_int8.shape == (num, dim)
    w = emb.weight.numpy()
    mn, mx = O.minmax(w, ch_axis=0)
    s, z = O.calc_qparams(mn, mx, True, -128, 127, True)
    codes = O.quantize(w, s, z, -128, 127, ch_axis=0)
    assert np.array_equal(q.weight_int8.numpy(), codes) and np.array_equal(q.weight_scale.numpy(), s)
    rng = np.random.default_rng(num)
    idx = rng.integers(0, num, (4, 37)).astype(idx_dtype)
    idx[0, :5] = 3
    y = q(hip(idx)).numpy()
    want = Br.embedding(codes, s, z, idx, padding_idx=3)
    assert y.shape == (4, 37, dim)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    # test_breadth.py:12-23
    yf = np.where((idx == 3)[..., None], 0, w[idx])
    assert np.abs(yf - y).mean() / (np.abs(yf).mean() + 1e-9) < 0.02
    # test_breadth.py:25-30
    assert q.weight_int8.numpy().nbytes + q.weight_scale.numpy().nbytes < num * dim * 4 / 2


def test_embedding_index_checks():
    q = nnq.Embedding.from_float(nn.Embedding(10, 8))
    with pytest.raises(IndexError, match=r"index 10 is out of range for a table with 10 entries"):
        q(hip(np.array([1, 10], np.int64)))
    with pytest.raises(IndexError, match=r"index -1 is out of range"):
        q(hip(np.array([-1, 2], np.int64)))
    with pytest.raises(TypeError, match="indices must be an integer tensor"):
        q(hip(np.array([1.0, 2.0], np.float32)))
    assert q(hip(np.zeros((0,), np.int64))).shape == (0, 8)


@pytest.mark.parametrize("mode", ["sum", "mean", "max"])
def test_embedding_bag_bit_exact(mode):
    bag = nn.EmbeddingBag(50, 16, mode=mode, padding_idx=9)
    q = nnq.EmbeddingBag.from_float(bag)
    codes, s, z = q.weight_int8.numpy(), q.weight_scale.numpy(), q.weight_zero_point.numpy()
    idx = np.array([1, 5, 9, 3, 7, 2, 8, 9, 9], np.int64)
    off = np.array([0, 3, 5, 5], np.int64)
    y = q(hip(idx), hip(off)).numpy()
    want = Br.embedding_bag(codes, s, z, idx, off, mode, padding_idx=9)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(y[2], np.zeros(16, np.float32))  # the empty bag
    # 2-d indices: every row a bag; int32 indices and offsets
    idx2 = np.random.default_rng(0).integers(0, 50, (64, 11)).astype(np.int32)
    y2 = q(hip(idx2)).numpy()
    assert np.array_equal(y2.view(np.uint32),
                          Br.embedding_bag(codes, s, z, idx2, None, mode, padding_idx=9).view(np.uint32))
    with pytest.raises(ValueError, match="offsets required"):
        q(hip(idx))


def test_convert_installs_embeddings_without_calibration():
    # test_breadth.py:32-35, test_module_breadth.py:91-104
    qm = Q.convert(Q.prepare(nn.Sequential(nn.Embedding(50, 16))))
    assert isinstance(qm[0], nnq.Embedding)
    m = nn.Sequential(nn.EmbeddingBag(50, 16, mode="mean"))
    w = m[0].weight.numpy()
    qm = Q.convert(m)
    assert isinstance(qm[0], nnq.EmbeddingBag) and qm[0].weight_int8.dtype is L.int8
    idx, off = np.array([1, 5, 9, 3, 7, 2, 8], np.int64), np.array([0, 3, 5], np.int64)
    yq = qm[0](hip(idx), hip(off)).numpy()
    yf = np.stack([w[[1, 5, 9]].mean(0), w[[3, 7]].mean(0), w[[2, 8]].mean(0)])
    assert np.abs(yf - yq).max() / (np.abs(yf).max() + 1e-9) < 0.05


def test_integer_input_passes_through_quantize():
    # test_breadth.py:38-47
    idx = hip(np.array([1, 2, 3], np.int64))
    quant = nnq.Quantize(hip(np.float32(0.05)), hip(np.float32(0.0)))
    assert np.array_equal(quant(idx).numpy(), [1, 2, 3])


# ---------------------------------------------------------------- activations
_ACTS = [(nn.Sigmoid, nnq.Sigmoid, Br.SIGMOID, {}), (nn.Hardswish, nnq.Hardswish, Br.HARDSWISH, {}),
         (nn.Hardsigmoid, nnq.Hardsigmoid, Br.HARDSIGMOID, {}), (nn.Tanh, nnq.Tanh, Br.TANH, {}),
         (nn.ELU, nnq.ELU, Br.ELU, {"alpha": 0.7}), (nn.LeakyReLU, nnq.LeakyReLU, Br.LEAKY_RELU, {"negative_slope": 0.2})]
_EXACT = (Br.HARDSWISH, Br.HARDSIGMOID, Br.LEAKY_RELU)


@pytest.mark.parametrize("fcls,qcls,kind,kw", _ACTS)
def test_float_activation(fcls, qcls, kind, kw):
    x = (np.random.default_rng(kind).standard_normal(100003) * 3).astype(np.float32)
    y = fcls(**kw)(hip(x)).numpy()
    want = Br.act(kind, x, *kw.values())
    if kind in _EXACT:
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    else:  # exp / tanh: library last bits differ
        assert np.abs(y - want).max() <= 4e-7 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("fcls,qcls,kind,kw", _ACTS)
def test_quantized_activation_on_codes_and_on_floats(fcls, qcls, kind, kw):
    rng = np.random.default_rng(10 + kind)
    alpha = next(iter(kw.values()), 0.0)
    x = (rng.standard_normal((8, 4099)) * 2).astype(np.float32)
    s, z = np.float32(16 / 255), np.float32(128)
    y_float = Br.act(kind, x, alpha)
    S = np.float32((y_float.max() - min(y_float.min(), 0)) / 255)
    Z = np.float32(np.rint(-min(y_float.min(), 0) / S))
    act = qcls(hip(S), hip(Z), Q.quint8)
    act._configure(fcls(**kw))
    # on codes
    xq = nnq.Quantize(hip(s), hip(z), Q.quint8)(hip(x))
    out = act(xq)
    assert out._grid is not None and out.shape == x.shape
    stored = O.quantize(x, s, z, 0, 255, code_offset=-128)
    want = Br.quantized_act_codes(kind, stored, -128, s, z, alpha, S, Z, 0, 255, -128)
    got = out._grid.codes.numpy()
    if kind in _EXACT:
        assert np.array_equal(got, want)
    else:
        d = np.abs(got.astype(np.int32) - want.astype(np.int32))
        assert d.max() <= 1 and (d != 0).mean() < 1e-3
    # on plain floats: activation + fake-quantize
    yf = act(hip(x)).numpy()
    want_f = Br.quantized_act(kind, x, alpha, S, Z, 0, 255)
    if kind in _EXACT:
        assert np.array_equal(yf.view(np.uint32), want_f.view(np.uint32))
    else:
        assert np.abs(yf - want_f).max() <= S * 1.001 and (yf != want_f).mean() < 1e-3


@pytest.mark.parametrize("fcls,qcls,kind,kw", _ACTS)
def test_convert_installs_quantized_activation(fcls, qcls, kind, kw):
    # test_module_breadth.py:55-89
    rng = np.random.default_rng(kind)
    m = nn.Sequential(nnq.QuantStub(), nn.Linear(64, 64), fcls(**kw), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    w, b = m[1].weight.numpy(), m[1].bias.numpy()
    alpha = next(iter(kw.values()), 0.0)
    for _ in range(5):
        x = rng.standard_normal((8, 64)).astype(np.float32)
        h = x @ w.T + b
        prepared[0].activation_post_process(hip(x))
        prepared[1].activation_post_process(hip(h))
        prepared[2].activation_post_process(hip(Br.act(kind, h, alpha)))
    qm = Q.convert(prepared)
    assert isinstance(qm[2], qcls)
    if kind == Br.LEAKY_RELU:
        assert qm[2].negative_slope == pytest.approx(0.2)
    x = rng.standard_normal((8, 64)).astype(np.float32)
    yq = qm(hip(x)).numpy()
    yf = Br.act(kind, x @ w.T + b, alpha)
    assert np.abs(yf - yq).max() / (np.abs(yf).max() + 1e-9) < 0.1


# ---------------------------------------------------------------- transposed convolution
@pytest.mark.parametrize("cin,cout,k,stride,padding,output_padding,dilation,groups",
                         [(8, 4, 3, 2, 1, 1, 1, 1),      # test_module_breadth.py:33-52
                          (32, 48, (3, 2), (2, 3), (1, 0), (1, 2), 1, 1),
                          (32, 32, 3, 1, 1, 0, 1, 2),     # stride 1: no zero insertion
                          (16, 24, 2, 2, 0, 0, (2, 1), 1)])
def test_conv_transpose2d(cin, cout, k, stride, padding, output_padding, dilation, groups):
    pair = lambda v: (v, v) if isinstance(v, int) else v
    rng = np.random.default_rng(cin + cout)
    m = nn.Sequential(nnq.QuantStub(), nn.ConvTranspose2d(cin, cout, k, stride=stride, padding=padding,
                                                          output_padding=output_padding, groups=groups,
                                                          dilation=dilation), nnq.DeQuantStub())
    w, b = m[1].weight.numpy(), m[1].bias.numpy()
    args = (pair(stride), pair(padding), pair(output_padding), pair(dilation), groups)
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(6):
        x = rng.standard_normal((2, cin, 8, 7)).astype(np.float32)
        prepared[0].activation_post_process(hip(x))
        prepared[1].activation_post_process(hip(Br.conv_transpose2d(x, w, b, *args).astype(np.float32)))
    qm = Q.convert(prepared)
    ct = qm[1]
    assert isinstance(ct, nnq.ConvTranspose2d) and ct.weight_int8.dtype is L.int8
    assert ct.weight_int8.shape == w.shape and ct.weight_scale.shape == (cout // groups,)
    x = rng.standard_normal((2, cin, 8, 7)).astype(np.float32)
    yf = Br.conv_transpose2d(x, w, b, *args)
    out = ct(qm[0](hip(x)))
    yq = qm(hip(x)).numpy()
    assert yq.shape == yf.shape
    assert np.abs(yf - yq).mean() / (np.abs(yf).mean() + 1e-9) < 0.05
    # the float64 scatter form on the dequantized operands, requantized: codes agree up to
    # one step on rounding ties
    s0, z0 = qm[0].scale.item(), qm[0].zero_point.item()
    xd = O.dequantize(O.quantize(x, s0, z0, 0, 255, code_offset=-128), s0, z0, code_offset=-128)
    ws = ct.weight_scale.numpy()
    wd = ct.weight_int8.numpy().astype(np.float32) * ws[None, :, None, None]
    ref = Br.conv_transpose2d(xd, wd, b, *args)
    S, Z = ct.scale.item(), ct.zero_point.item()
    want = np.clip(np.rint(ref / np.float64(S)) + Z, 0, 255)
    got = np.transpose(out._grid.codes.numpy().astype(np.int32) + 128, (0, 3, 1, 2))
    d = np.abs(got - want)
    assert d.max() <= 1 and (d != 0).mean() < 0.01


# ---------------------------------------------------------------- dynamic LSTM
def _oracle_lstm_stack(q, x, hx, batch_first):
    """Layer by layer, direction by direction, with Br.lstm on the dequantized weights."""
    import lucid_amd.nn.quantized.dynamic as nnqd  # noqa: F401
    H, dirs = q.hidden_size, 2 if q.bidirectional else 1
    xs = np.transpose(x, (1, 0, 2)) if batch_first else x
    Tn, Bn, _ = xs.shape
    hs, cs = [], []
    for k in range(q.num_layers):
        outs = []
        for d, suffix in enumerate(("", "_reverse")[:dirs]):
            def w(name):
                return (getattr(q, name + "_int8").numpy().astype(np.float32) *
                        getattr(q, name + "_scale").numpy()[:, None]).astype(np.float32)
            wih, whh = w(f"weight_ih_l{k}{suffix}"), w(f"weight_hh_l{k}{suffix}")
            if q.bias:
                bih, bhh = (getattr(q, f"bias_{n}_l{k}{suffix}").numpy() for n in ("ih", "hh"))
            else:
                bih = bhh = np.zeros(4 * H, np.float32)
            idx = k * dirs + d
            h0 = hx[0][idx] if hx is not None else np.zeros((Bn, H), np.float32)
            c0 = hx[1][idx] if hx is not None else np.zeros((Bn, H), np.float32)
            seq = xs[::-1] if d == 1 else xs
            y, hn, cn = Br.lstm(seq, h0, c0, wih, whh, bih, bhh)
            outs.append(y[::-1] if d == 1 else y)
            hs.append(hn)
            cs.append(cn)
        xs = np.concatenate(outs, axis=-1)
    y = np.transpose(xs, (1, 0, 2)) if batch_first else xs
    return y, np.stack(hs), np.stack(cs)


@pytest.mark.parametrize("layers,bidir,batch_first,bias,with_state",
                         [(1, False, True, True, False), (2, True, False, True, True), (2, False, True, False, True)])
def test_dynamic_lstm(layers, bidir, batch_first, bias, with_state):
    import lucid_amd.nn.quantized.dynamic as nnqd
    rng = np.random.default_rng(layers * 7 + bidir)
    I, H, Bn, Tn = 8, 16, 4, 5
    lstm = nn.LSTM(I, H, num_layers=layers, bias=bias, batch_first=batch_first, bidirectional=bidir)
    qm = Q.quantize_dynamic(lstm)
    assert isinstance(qm, nnqd.LSTM) and qm.weight_ih_l0_int8.dtype is L.int8
    # test_dynamic_ptq.py:55-64: the state dict holds the int8 form only
    assert [k for k in qm.state_dict() if k.startswith("weight_ih_l0")][:2] == ["weight_ih_l0_int8", "weight_ih_l0_scale"]
    assert not any(k in qm.state_dict() for k in ("weight_ih_l0", "weight_hh_l0"))
    x = rng.standard_normal((Bn, Tn, I) if batch_first else (Tn, Bn, I)).astype(np.float32)
    dirs = 2 if bidir else 1
    hx = None
    if with_state:
        hx = tuple(rng.standard_normal((layers * dirs, Bn, H)).astype(np.float32) for _ in range(2))
    y, (hn, cn) = qm(hip(x), None if hx is None else (hip(hx[0]), hip(hx[1])))
    wy, wh, wc = _oracle_lstm_stack(qm, x, hx, batch_first)
    assert y.shape == wy.shape and hn.shape == wh.shape
    for got, want in ((y.numpy(), wy), (hn.numpy(), wh), (cn.numpy(), wc)):
        assert np.abs(got - want).max() < 2e-5
    # test_dynamic_ptq.py:66-75: close to the float LSTM (float weights through the same recurrence)
    fl = {n: t.numpy() for n, t in lstm.named_parameters()}

    class F:  # the float weights presented as a "quantized" module with unit scales
        pass
    f = F()
    f.hidden_size, f.bidirectional, f.num_layers, f.bias = H, bidir, layers, bias
    for n, v in fl.items():
        if n.startswith("weight"):
            setattr(f, n + "_int8", type("A", (), {"numpy": lambda self, v=v: v})())
            setattr(f, n + "_scale", type("A", (), {"numpy": lambda self, v=v: np.ones(v.shape[0], np.float32)})())
        else:
            setattr(f, n, type("A", (), {"numpy": lambda self, v=v: v})())
    yf, _, _ = _oracle_lstm_stack(f, x, hx, batch_first)
    assert np.abs(yf - y.numpy()).mean() / (np.abs(yf).mean() + 1e-9) < 0.03


def _deq(q, name):
    return (getattr(q, name + "_int8").numpy().astype(np.float32) *
            getattr(q, name + "_scale").numpy()[:, None]).astype(np.float32)


@pytest.mark.parametrize("layers,bidir,proj,sorted_input", [(1, False, 0, True), (2, True, 0, False), (1, False, 6, True),
                                                            (2, True, 5, False)])
def test_dynamic_lstm_packed_sequences_and_projection(layers, bidir, proj, sorted_input):
    """PackedSequence input and proj_size (lucid/nn/quantized/dynamic/rnn.py:66-84 hands both to
    the float shell, lucid/nn/modules/rnn.py:585-795): against the oracle's recurrence run with
    the packed active-set schedule, layer by layer and direction by direction."""
    import lucid_amd.nn.quantized.dynamic as nnqd
    from lucid_amd.nn.utils.rnn import PackedSequence, pack_padded_sequence, pad_packed_sequence
    rng = np.random.default_rng(layers * 5 + bidir + proj)
    I, H, Bn, Tn = 8, 16, 5, 7
    R = proj if proj else H
    dirs = 2 if bidir else 1
    lengths = [7, 5, 5, 2, 1] if sorted_input else [2, 7, 1, 5, 5]
    lstm = nn.LSTM(I, H, num_layers=layers, bidirectional=bidir, proj_size=proj)
    qm = Q.quantize_dynamic(lstm)
    assert isinstance(qm, nnqd.LSTM) and qm.proj_size == proj
    if proj:
        assert qm.weight_hr_l0_int8.shape == (proj, H) and qm.weight_hh_l0_int8.shape == (4 * H, proj)
    x = rng.standard_normal((Tn, Bn, I)).astype(np.float32)
    packed = pack_padded_sequence(hip(x), lengths, enforce_sorted=sorted_input)
    assert isinstance(packed, PackedSequence) and packed.data.shape == (sum(lengths), I)
    # the packing itself, against numpy
    order = sorted(range(Bn), key=lambda i: -lengths[i])
    slen = [lengths[i] for i in order]
    bsz = [sum(1 for v in slen if v > t) for t in range(Tn)]
    want = np.concatenate([x[t, order[:bs]] for t, bs in enumerate(bsz)])
    assert np.array_equal(packed.data.numpy(), want) and packed.batch_sizes.numpy().tolist() == bsz
    hx = (rng.standard_normal((layers * dirs, Bn, R)).astype(np.float32),
          rng.standard_normal((layers * dirs, Bn, H)).astype(np.float32))
    out, (hn, cn) = qm(packed, (hip(hx[0]), hip(hx[1])))
    assert isinstance(out, PackedSequence) and out.data.shape == (sum(lengths), dirs * R)
    # oracle: padded in packed order, the schedule, states as given; final states back in caller order
    xs = np.zeros((Tn, Bn, I), np.float32)
    off = 0
    for t, bs in enumerate(bsz):
        xs[t, :bs] = want[off:off + bs]
        off += bs
    hs, cs = [], []
    for k in range(layers):
        outs = []
        for d, suffix in enumerate(("", "_reverse")[:dirs]):
            idx = k * dirs + d
            y, h, c = Br.lstm(xs, hx[0][idx], hx[1][idx], _deq(qm, f"weight_ih_l{k}{suffix}"),
                              _deq(qm, f"weight_hh_l{k}{suffix}"), getattr(qm, f"bias_ih_l{k}{suffix}").numpy(),
                              getattr(qm, f"bias_hh_l{k}{suffix}").numpy(),
                              w_hr=_deq(qm, f"weight_hr_l{k}{suffix}") if proj else None, batch_sizes=bsz, reverse=d == 1)
            outs.append(y)
            hs.append(h)
            cs.append(c)
        xs = np.concatenate(outs, axis=-1)
    wy = np.concatenate([xs[t, :bs] for t, bs in enumerate(bsz)])
    inv = packed.unsorted_indices.numpy().tolist()
    wh, wc = np.stack(hs)[:, inv], np.stack(cs)[:, inv]
    for got, exp in ((out.data.numpy(), wy), (hn.numpy(), wh), (cn.numpy(), wc)):
        assert got.shape == exp.shape and np.abs(got - exp).max() < 2e-5
    # unpacking restores the caller's order and lengths
    padded, lens = pad_packed_sequence(out, total_length=Tn)
    assert lens.numpy().tolist() == lengths
    for b, n in enumerate(lengths):
        assert np.abs(padded.numpy()[:n, b] - xs[:n, inv[b]]).max() < 2e-5 and not padded.numpy()[n:, b].any()
    # a dense tensor through the same module still takes the dense route
    yd, _ = qm(hip(x))
    assert yd.shape == (Tn, Bn, dirs * R)


def test_pack_and_pad_round_trip_on_both_devices():
    from lucid_amd.nn.utils.rnn import pack_padded_sequence, pack_sequence, pad_packed_sequence, pad_sequence
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 6, 3)).astype(np.float32)            # batch-first (B, T, F)
    lengths = [3, 6, 1, 4]
    for dev in ("cpu", "hip"):
        p = pack_padded_sequence(L.tensor(x, device=dev), lengths, batch_first=True, enforce_sorted=False)
        back, lens = pad_packed_sequence(p, batch_first=True, padding_value=-1.0)
        assert lens.numpy().tolist() == lengths and back.shape == (4, 6, 3) and back.device == dev
        for b, n in enumerate(lengths):
            assert np.array_equal(back.numpy()[b, :n], x[b, :n]) and (back.numpy()[b, n:] == -1.0).all()
    with pytest.raises(ValueError, match="sorted"):
        pack_padded_sequence(L.tensor(x), lengths, batch_first=True)
    seqs = [L.tensor(rng.standard_normal((n, 2)).astype(np.float32)) for n in (5, 3, 2)]
    assert pad_sequence(seqs).shape == (5, 3, 2)
    assert pack_sequence(seqs).batch_sizes.numpy().tolist() == [3, 3, 2, 1, 1]


# ---------------------------------------------------------------- Conv1d
@pytest.mark.parametrize("cin,cout,k,stride,padding,dilation,groups,Ln",
                         [(16, 32, 3, 1, 1, 1, 1, 50), (32, 48, 5, 2, 2, 1, 1, 37), (32, 32, 3, 1, "same", 2, 2, 64),
                          (16, 16, 1, 1, 0, 1, 1, 9), (64, 64, 7, 3, "valid", 1, 4, 100)])
def test_conv1d_bit_exact_against_the_oracle(cin, cout, k, stride, padding, dilation, groups, Ln):
    """nnq.Conv1d == the oracle's integer convolution of the same codes as a one-row image
    (conv.py:232-385 on the 2-d kernel), codes bit for bit; the float view within a step."""
    rng = np.random.default_rng(cin * 3 + cout + k)
    m = nn.Sequential(nnq.QuantStub(), nn.Conv1d(cin, cout, k, stride=stride, padding=padding, dilation=dilation,
                                                 groups=groups), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(4):
        x = rng.standard_normal((3, cin, Ln)).astype(np.float32)
        prepared[0].activation_post_process(hip(x))
        prepared[1].activation_post_process(hip((rng.standard_normal((3, cout, 4)) * 2).astype(np.float32)))
    qm = Q.convert(prepared)
    c1 = qm[1]
    assert isinstance(c1, nnq.Conv1d) and c1.weight_int8.shape == (cout, cin // groups, k)
    x = rng.standard_normal((3, cin, Ln)).astype(np.float32)
    xq = qm[0](hip(x))
    out = c1(xq)
    # the same layer through the oracle: NHWC codes of a (B, 1, L, C) image, OHWI weights
    s0, z0 = qm[0].scale.item(), qm[0].zero_point.item()
    codes = O.quantize(x, s0, z0, 0, 255, code_offset=-128)                      # (B, C, L)
    x_nhwc = np.ascontiguousarray(np.transpose(codes, (0, 2, 1))[:, None, :, :])  # (B, 1, L, C)
    w_ohwi = np.ascontiguousarray(np.transpose(c1.weight_int8.numpy(), (0, 2, 1))[:, None, :, :])
    if padding == "same":
        total = max(0, (-(-Ln // stride) - 1) * stride + (k - 1) * dilation + 1 - Ln)
        pad = (0, 0, total // 2, total - total // 2)
    elif padding == "valid":
        pad = (0, 0, 0, 0)
    else:
        pad = (0, 0, padding, padding)
    want = O.qconv2d(x_nhwc, w_ohwi, int(z0) - 128, np.float32(s0), c1.weight_scale.numpy(), stride=(1, stride),
                     pad=pad, dilation=(1, dilation), groups=groups, bias=c1.bias.numpy(), out_mode=O.OUT_REQUANT_I8,
                     out_scale=np.float32(c1.scale.item()), out_zp=np.float32(c1.zero_point.item()), out_qmin=0,
                     out_qmax=255, out_offset=-128)                                # (B, 1, Lo, Cout)
    got = out._grid.codes.numpy()                                                  # (B, Cout, Lo)
    assert got.shape == (3, cout, want.shape[2])
    assert np.array_equal(got, np.transpose(want[:, 0], (0, 2, 1)))
    y = qm(hip(x)).numpy()
    assert y.shape == got.shape and np.isfinite(y).all()


@pytest.mark.parametrize("cin,cout,k,stride,padding,output_padding,dilation,groups",
                         [(16, 32, 3, 2, 1, 1, 1, 1), (32, 32, 4, 3, 0, 2, 1, 2), (16, 16, 3, 1, 1, 0, 2, 1)])
def test_conv_transpose1d(cin, cout, k, stride, padding, output_padding, dilation, groups):
    """nnq.ConvTranspose1d == nnq.ConvTranspose2d on the same operands as a one-row image, codes
    bit for bit (conv_transpose.py:162-319); the 2-d layer is checked against the oracle above."""
    rng = np.random.default_rng(cin + cout + k)
    m = nn.Sequential(nnq.QuantStub(), nn.ConvTranspose1d(cin, cout, k, stride=stride, padding=padding,
                                                          output_padding=output_padding, groups=groups,
                                                          dilation=dilation), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(4):
        prepared[0].activation_post_process(hip(rng.standard_normal((2, cin, 21)).astype(np.float32)))
        prepared[1].activation_post_process(hip((rng.standard_normal((2, cout, 5)) * 0.7).astype(np.float32)))
    qm = Q.convert(prepared)
    c1 = qm[1]
    assert isinstance(c1, nnq.ConvTranspose1d) and c1.weight_int8.shape == (cin, cout // groups, k)
    c2 = nnq.ConvTranspose2d(cin, cout, (1, k), (1, stride), (0, padding), (0, output_padding), (1, dilation), groups)
    c2.register_buffer("weight_int8", L.tensor(c1.weight_int8.numpy()[:, :, None, :], device="hip"))
    for name in ("weight_scale", "weight_zero_point", "bias", "scale", "zero_point"):
        c2.register_buffer(name, getattr(c1, name))
    c2.out_qdtype = c1.out_qdtype
    x = rng.standard_normal((2, cin, 21)).astype(np.float32)
    y1 = c1(qm[0](hip(x)))
    # the 2-d layer on the same codes: quantize the (B, C, 1, L) view with the same stub
    y2 = c2(qm[0](hip(x[:, :, None, :])))
    got = y1._grid.codes.numpy()                                   # (B, Cout, Lo)
    want = np.transpose(y2._grid.codes.numpy()[:, 0], (0, 2, 1))   # NHWC (B, 1, Lo, Cout) -> (B, Cout, Lo)
    lo = (21 - 1) * stride - 2 * padding + dilation * (k - 1) + output_padding + 1
    assert got.shape == (2, cout, lo) and np.array_equal(got, want)
    assert np.isfinite(qm(hip(x)).numpy()).all()


# ---------------------------------------------------------------- Conv3d
@pytest.mark.parametrize("cin,cout,k,stride,padding,dilation,groups,vol",
                         [(16, 32, 3, 1, 1, 1, 1, (6, 10, 12)), (8, 24, (1, 3, 2), (1, 2, 1), (0, 1, 1), 1, 1, (4, 9, 7)),
                          (32, 32, 3, (2, 1, 1), "same", (1, 2, 1), 2, (5, 8, 8)), (16, 16, 1, 1, 0, 1, 1, (3, 4, 5)),
                          (48, 96, (2, 3, 3), 2, "valid", 1, 3, (6, 11, 9))])
def test_conv3d_bit_exact_against_the_oracle(cin, cout, k, stride, padding, dilation, groups, vol):
    """nnq.Conv3d (conv.py:545-700) == the oracle's integer Conv3d of the same codes, bit for
    bit; the float view lies on the output grid."""
    import oracle.breadth as Br
    three = lambda v: (v,) * 3 if isinstance(v, int) else tuple(v)
    rng = np.random.default_rng(cin * 3 + cout + sum(vol))
    m = nn.Sequential(nnq.QuantStub(), nn.Conv3d(cin, cout, k, stride=stride, padding=padding, dilation=dilation,
                                                 groups=groups), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(4):
        x = rng.standard_normal((2, cin, *vol)).astype(np.float32)
        prepared[0].activation_post_process(hip(x))
        prepared[1].activation_post_process(hip((rng.standard_normal((2, cout, 2, 2, 2)) * 1.5).astype(np.float32)))
    qm = Q.convert(prepared)
    c3 = qm[1]
    assert isinstance(c3, nnq.Conv3d) and c3.weight_int8.shape == (cout, cin // groups, *three(k))
    x = rng.standard_normal((2, cin, *vol)).astype(np.float32)
    out = c3(qm[0](hip(x)))
    s0, z0 = qm[0].scale.item(), qm[0].zero_point.item()
    codes = O.quantize(x, s0, z0, 0, 255, code_offset=-128)
    K3, S3, D3 = three(k), three(stride), three(dilation)
    if padding == "same":
        pad = []
        for n, kk, ss, dd in zip(vol, K3, S3, D3):
            total = max(0, (-(-n // ss) - 1) * ss + (kk - 1) * dd + 1 - n)
            pad.append((total // 2, total - total // 2))
    elif padding == "valid":
        pad = [(0, 0)] * 3
    else:
        pad = [(p, p) for p in three(padding)]
    want = Br.qconv3d(codes, c3.weight_int8.numpy(), int(z0) - 128, np.float32(s0), c3.weight_scale.numpy(),
                      stride=S3, pad=tuple(pad), dilation=D3, groups=groups, bias=c3.bias.numpy(),
                      out_mode=O.OUT_REQUANT_I8, out_scale=np.float32(c3.scale.item()),
                      out_zp=np.float32(c3.zero_point.item()), out_qmin=0, out_qmax=255, out_offset=-128)
    got = volume_codes(out)
    assert out._grid.layout == ("nhwc" if (cin // groups) % 16 == 0 else "plain")
    assert got.shape == want.shape and np.array_equal(got, want)
    assert len(np.unique(got)) > 20
    y = qm(hip(x)).numpy()
    exp_y = (want.astype(np.float32) + 128 - np.float32(c3.zero_point.item())) * np.float32(c3.scale.item())
    assert np.array_equal(y, exp_y)


GATHER3D_CASES = [
    # B, C, Co, vol, kernel, stride, pads, dilation, groups, tile shape
    (2, 16, 32, (5, 9, 11), (3, 3, 3), (1, 1, 1), ((1, 1), (1, 1), (1, 1)), (1, 1, 1), 1, 0),
    (1, 32, 24, (4, 13, 7), (2, 3, 1), (2, 1, 2), ((0, 1), (2, 0), (0, 0)), (1, 2, 1), 1, 5),
    (3, 64, 64, (6, 10, 10), (3, 3, 3), (1, 2, 1), ((1, 1), (0, 1), (2, 2)), (2, 1, 1), 1, 6),
    (2, 96, 160, (3, 8, 9), (1, 3, 3), (1, 1, 1), ((0, 0), (1, 1), (1, 1)), (1, 1, 1), 2, 3),
    (2, 48, 288, (4, 6, 6), (3, 1, 2), (1, 1, 1), ((2, 2), (0, 0), (1, 0)), (1, 1, 3), 3, 4),
    (1, 16, 16, (2, 3, 3), (2, 2, 2), (1, 1, 1), ((0, 0), (0, 0), (0, 0)), (1, 1, 1), 1, 9),
    (2, 32, 48, (7, 7, 7), (3, 3, 3), (2, 2, 2), ((1, 1), (1, 1), (1, 1)), (1, 1, 1), 1, 9),
    # shape 15: the box-of-outputs kernel with the input halo in LDS (stride 1, 64-channel slices)
    (2, 64, 64, (6, 10, 10), (3, 3, 3), (1, 1, 1), ((1, 1), (1, 1), (1, 1)), (1, 1, 1), 1, 15),
    (1, 128, 80, (5, 9, 21), (2, 3, 3), (1, 1, 1), ((0, 1), (2, 0), (1, 1)), (2, 1, 2), 2, 15),
    (2, 128, 32, (3, 5, 4), (3, 1, 2), (1, 1, 1), ((1, 1), (0, 0), (0, 1)), (1, 1, 1), 1, 15),
]


@pytest.mark.parametrize("B,C,Co,vol,kernel,stride,pads,dilation,groups,shape", GATHER3D_CASES)
def test_conv3d_loader_gather_exact(B, C, Co, vol, kernel, stride, pads, dilation, groups, shape):
    """lq_qconv3d_i8 (taps gathered by the tile loader from NDHWC codes) against the oracle's
    integer Conv3d: raw accumulators, the requantize epilogue with bias and ReLU, and float32
    output, on strides, dilations, one-sided pads, groups and every tile shape that has the gather."""
    from lucid_amd import _ops
    rng = np.random.default_rng(B * 100 + C + Co + sum(vol) + shape)
    Cg = C // groups
    x = rng.integers(-128, 128, (B, C, *vol), dtype=np.int8)
    w = rng.integers(-127, 128, (Co, Cg, *kernel), dtype=np.int8)
    a_zp = int(rng.integers(-100, 100))
    a_scale = np.float32(0.021)
    w_scale = rng.uniform(0.001, 0.01, Co).astype(np.float32)
    bias = (rng.standard_normal(Co) * 0.5).astype(np.float32)
    xl = hip(np.ascontiguousarray(np.transpose(x, (0, 2, 3, 4, 1))))
    wl = hip(np.ascontiguousarray(np.transpose(w, (0, 2, 3, 4, 1))))
    wsum = hip(w.reshape(Co, -1).astype(np.int32).sum(1).astype(np.int32))
    common = dict(stride=stride, pad=pads, dilation=dilation, groups=groups)
    to_ncdhw = lambda t: np.ascontiguousarray(np.moveaxis(t.numpy(), -1, 1))
    acc = _ops.qconv3d_i8(xl, wl, a_zp=a_zp, out_mode=_ops.OUT_ACC_I32, tile_config=shape, **common)
    want_acc = Br.qconv3d(x, w, a_zp, a_scale, w_scale, out_mode=O.OUT_ACC_I32, **common)
    assert np.array_equal(to_ncdhw(acc), want_acc)
    k = Cg * kernel[0] * kernel[1] * kernel[2]
    out_scale = np.float32(0.0135 * np.sqrt(k))  # ~6 standard deviations of the float result over the grid
    got = _ops.qconv3d_i8(xl, wl, a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum, bias=hip(bias),
                          relu=True, out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(out_scale), out_zp=hip(np.float32(3.0)),
                          out_qmin=0, out_qmax=255, out_offset=-128, tile_config=shape, **common)
    want = Br.qconv3d(x, w, a_zp, a_scale, w_scale, bias=bias, relu=True, out_mode=O.OUT_REQUANT_I8, out_scale=out_scale,
                      out_zp=np.float32(3.0), out_qmin=0, out_qmax=255, out_offset=-128, **common)
    assert np.array_equal(to_ncdhw(got), want)
    assert want.size < 1000 or len(np.unique(want)) > 20
    f = _ops.qconv3d_i8(xl, wl, a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum, bias=hip(bias),
                        out_mode=_ops.OUT_F32, tile_config=shape, **common)
    want_f = Br.qconv3d(x, w, a_zp, a_scale, w_scale, bias=bias, out_mode=O.OUT_F32, **common)
    assert np.array_equal(to_ncdhw(f).view(np.uint32), want_f.view(np.uint32))


def test_conv3d_loader_gather_affine_filters_and_refusals():
    """Affine filter codes through lq_qconv3d_i8 (window sums from an all-ones filter) against
    the oracle; channel counts the gather is not built for are refused by name."""
    from lucid_amd import _C, _ops
    rng = np.random.default_rng(77)
    B, C, Co, vol, kernel = 2, 32, 40, (4, 6, 5), (3, 2, 3)
    x = rng.integers(-128, 128, (B, C, *vol), dtype=np.int8)
    w = rng.integers(-128, 128, (Co, C, *kernel), dtype=np.int8)
    w_zp = rng.integers(-20, 20, Co).astype(np.int32)
    a_zp, a_scale = -7, np.float32(0.03)
    w_scale = rng.uniform(0.001, 0.01, Co).astype(np.float32)
    pads = ((1, 0), (0, 1), (1, 1))
    xl = hip(np.ascontiguousarray(np.transpose(x, (0, 2, 3, 4, 1))))
    wl = hip(np.ascontiguousarray(np.transpose(w, (0, 2, 3, 4, 1))))
    wsum = hip(w.reshape(Co, -1).astype(np.int32).sum(1).astype(np.int32))
    got = _ops.qconv3d_i8(xl, wl, a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum, pad=pads,
                          out_mode=_ops.OUT_F32, w_zp=hip(w_zp))
    want = Br.qconv3d(x, w, a_zp, a_scale, w_scale, pad=pads, out_mode=O.OUT_F32, w_zp=w_zp)
    assert np.array_equal(np.moveaxis(got.numpy(), -1, 1).view(np.uint32), want.view(np.uint32))
    with pytest.raises(NotImplementedError, match=r"Cin/groups % 16 == 0 \(got 8\)"):
        _ops.qconv3d_i8(hip(np.zeros((1, 2, 2, 2, 8), np.int8)), hip(np.zeros((4, 1, 1, 1, 8), np.int8)), a_zp=0,
                        out_mode=_ops.OUT_ACC_I32)
    with pytest.raises(NotImplementedError, match="no volumetric gather"):
        _ops.qconv3d_i8(hip(np.zeros((1, 2, 2, 2, 16), np.int8)), hip(np.zeros((4, 1, 1, 1, 16), np.int8)), a_zp=0,
                        out_mode=_ops.OUT_ACC_I32, tile_config=1)
    with pytest.raises(_C.ShapeMismatch, match="empty output"):
        _ops.qconv3d_i8(hip(np.zeros((1, 2, 2, 2, 16), np.int8)), hip(np.zeros((4, 3, 1, 1, 16), np.int8)), a_zp=0,
                        out_mode=_ops.OUT_ACC_I32)


def test_conv3d_refuses_what_it_does_not_do():
    c3 = nnq.Conv3d(4, 4, 3)
    c3.padding_mode = "mirror"
    x = nnq.Quantize(hip(np.float32(0.1)), hip(np.float32(128.0)), Q.quint8)(hip(np.zeros((1, 4, 3, 3, 3), np.float32)))
    with pytest.raises(ValueError, match="padding_mode"):
        c3(x)
    with pytest.raises(Exception):
        nnq.Conv3d(4, 4, 3)(nnq.Quantize(hip(np.float32(0.1)), hip(np.float32(128.0)), Q.quint8)(
            hip(np.zeros((1, 4, 3, 3), np.float32))))


@pytest.mark.parametrize("cin,cout,k,stride,padding,output_padding,dilation,groups,vol",
                         [(16, 32, 3, 2, 1, 1, 1, 1, (3, 5, 4)), (32, 32, (2, 3, 2), (1, 3, 2), (0, 1, 0), (0, 2, 1), 1, 2, (4, 3, 5)),
                          (16, 16, 3, 1, 1, 0, (2, 1, 2), 1, (5, 4, 6))])
def test_conv_transpose3d_bit_exact_against_the_oracle(cin, cout, k, stride, padding, output_padding, dilation, groups,
                                                       vol):
    """nnq.ConvTranspose3d (conv_transpose.py:484-640) == the oracle's integer formulation
    (itself pinned against the scatter definition), codes bit for bit."""
    import oracle.breadth as Br
    three = lambda v: (v,) * 3 if isinstance(v, int) else tuple(v)
    rng = np.random.default_rng(cin + cout + sum(vol))
    m = nn.Sequential(nnq.QuantStub(), nn.ConvTranspose3d(cin, cout, k, stride=stride, padding=padding,
                                                          output_padding=output_padding, groups=groups,
                                                          dilation=dilation), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(4):
        prepared[0].activation_post_process(hip(rng.standard_normal((2, cin, *vol)).astype(np.float32)))
        prepared[1].activation_post_process(hip((rng.standard_normal((2, cout, 2, 2, 2)) * 0.8).astype(np.float32)))
    qm = Q.convert(prepared)
    t3 = qm[1]
    assert isinstance(t3, nnq.ConvTranspose3d) and t3.weight_int8.shape == (cin, cout // groups, *three(k))
    x = rng.standard_normal((2, cin, *vol)).astype(np.float32)
    out = t3(qm[0](hip(x)))
    s0, z0 = qm[0].scale.item(), qm[0].zero_point.item()
    codes = O.quantize(x, s0, z0, 0, 255, code_offset=-128)
    want = Br.qconv_transpose3d(codes, t3.weight_int8.numpy(), int(z0) - 128, np.float32(s0), t3.weight_scale.numpy(),
                                stride=three(stride), padding=three(padding), output_padding=three(output_padding),
                                dilation=three(dilation), groups=groups, bias=t3.bias.numpy(),
                                out_mode=O.OUT_REQUANT_I8, out_scale=np.float32(t3.scale.item()),
                                out_zp=np.float32(t3.zero_point.item()), out_qmin=0, out_qmax=255, out_offset=-128)
    got = volume_codes(out)
    size = [(n - 1) * s - 2 * p + d * (kk - 1) + op + 1 for n, s, p, d, kk, op in
            zip(vol, three(stride), three(padding), three(dilation), three(k), three(output_padding))]
    assert got.shape == (2, cout, *size) == want.shape
    assert np.array_equal(got, want)
    assert len(np.unique(got)) > 20
    assert np.isfinite(qm(hip(x)).numpy()).all()


@pytest.mark.parametrize("batches,R,Cn,pad_src,pad_dst", [(1, 64, 64, 0, 0), (3, 70, 130, 0, 0), (2, 1, 257, 5, 0),
                                                           (4, 200, 3, 0, 96), (2, 129, 65, 7, 33)])
def test_batched_byte_transpose(batches, R, Cn, pad_src, pad_dst):
    """lq_transpose_i8: every batch's R x Cn matrix becomes Cn x R, batch strides respected on
    both sides (the gap bytes of the destination keep what they held), edge tiles included."""
    from lucid_amd import _C
    rng = np.random.default_rng(R * 7 + Cn)
    ss, ds = R * Cn + pad_src, R * Cn + pad_dst
    src = rng.integers(-128, 128, batches * ss).astype(np.int8)
    dst0 = rng.integers(-128, 128, batches * ds).astype(np.int8)
    s, d = hip(src), hip(dst0)
    _C.call("lq_transpose_i8", s.data_ptr, d.data_ptr, batches, R, Cn, ss, ds, None)
    got = d.numpy()
    want = dst0.copy()
    for b in range(batches):
        want[b * ds:b * ds + R * Cn] = src[b * ss:b * ss + R * Cn].reshape(R, Cn).T.ravel()
    assert np.array_equal(got, want)
    with pytest.raises(Exception):
        _C.call("lq_transpose_i8", s.data_ptr, d.data_ptr, batches, R, Cn, R * Cn - 1, ds, None)


@pytest.mark.parametrize("padding_mode", ["reflect", "replicate", "circular"])
def test_conv3d_with_a_padding_mode(padding_mode):
    """nnq.Conv3d with padding_mode != zeros (lucid/nn/quantized/conv.py:545; the float layer
    pre-pads with F.pad and convolves with padding 0, nn/modules/conv.py:104-123): the padded
    codes equal numpy's pad of the codes, the convolution equals the oracle on them."""
    rng = np.random.default_rng(20)
    B, Cc, D, H, W, Co = 2, 16, 4, 6, 5, 24
    codes = rng.integers(0, 256, (B, Cc, D, H, W)).astype(np.int16)
    wq = rng.integers(-127, 128, (Co, Cc, 3, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, Co).astype(np.float32)
    bias = rng.standard_normal(Co).astype(np.float32)
    conv = nnq.Conv3d(Cc, Co, 3, padding=(1, 2, 1))
    conv.padding_mode = padding_mode
    state = {"weight_int8": wq, "weight_scale": ws, "weight_zero_point": np.zeros(Co, np.float32), "bias": bias,
             "scale": np.float32(0.05), "zero_point": np.float32(120.0)}
    conv.load_state_dict({k: L.tensor(v, device="hip") for k, v in state.items()})
    from lucid_amd._tensor import Grid, Tensor
    in_scale, in_zp = np.float32(0.02), 128
    grid = Grid(hip((codes - 128).astype(np.int8)), hip(np.float32(in_scale)), hip(np.float32(in_zp)), Q.quint8, -128,
                in_zp, "plain")
    y = conv(Tensor.on_grid((B, Cc, D, H, W), grid))
    got = volume_codes(y)
    np_mode = {"reflect": "reflect", "replicate": "edge", "circular": "wrap"}[padding_mode]
    xp = np.pad((codes - 128).astype(np.int8), ((0, 0), (0, 0), (1, 1), (2, 2), (1, 1)), mode=np_mode)
    exp = Br.qconv3d(xp, wq, in_zp - 128, in_scale, ws, bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=0.05, out_zp=120.0,
                     out_qmin=0, out_qmax=255, out_offset=-128)
    assert got.shape == exp.shape and np.array_equal(got, exp)


def test_volumes_stay_channels_last_between_layers():
    """QuantStub -> Conv3d -> Conv3d (reflect padding) -> ConvTranspose3d -> DeQuantStub on a video
    batch: the stub and the first convolution leave channels-last codes, the padded layer and the
    transposed convolution take them in either order, the float view comes out in (B, C, D, H, W)
    order - all equal to the oracle chained layer by layer."""
    rng = np.random.default_rng(31)
    m = nn.Sequential(nnq.QuantStub(), nn.Conv3d(16, 32, 3, padding=1), nn.Conv3d(32, 16, (1, 3, 3), padding=(0, 1, 1)),
                      nn.ConvTranspose3d(16, 8, 2, stride=2), nnq.DeQuantStub())
    prepared = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(3):
        prepared[0].activation_post_process(hip(rng.standard_normal((2, 16, 4, 6, 5)).astype(np.float32)))
        for i, c in ((1, 32), (2, 16), (3, 8)):
            prepared[i].activation_post_process(hip((rng.standard_normal((2, c, 2, 2, 2)) * 1.2).astype(np.float32)))
    qm = Q.convert(prepared)
    qm[2].padding_mode = "reflect"
    x = rng.standard_normal((2, 16, 4, 6, 5)).astype(np.float32)
    q0 = qm[0](hip(x))
    assert q0._grid.layout == "nhwc" and q0._grid.codes.shape == (2, 4, 6, 5, 16)
    s0, z0 = qm[0].scale.item(), qm[0].zero_point.item()
    codes = O.quantize(x, s0, z0, 0, 255, code_offset=-128)
    assert np.array_equal(volume_codes(q0), codes)
    assert np.array_equal(q0.numpy(), (codes.astype(np.float32) + 128 - np.float32(z0)) * np.float32(s0))

    def req(mod):
        return dict(out_mode=O.OUT_REQUANT_I8, out_scale=np.float32(mod.scale.item()),
                    out_zp=np.float32(mod.zero_point.item()), out_qmin=0, out_qmax=255, out_offset=-128)

    y1 = qm[1](q0)
    assert y1._grid.layout == "nhwc"
    w1 = Br.qconv3d(codes, qm[1].weight_int8.numpy(), int(z0) - 128, np.float32(s0), qm[1].weight_scale.numpy(),
                    pad=((1, 1),) * 3, bias=qm[1].bias.numpy(), **req(qm[1]))
    assert np.array_equal(volume_codes(y1), w1)
    y2 = qm[2](y1)
    z1 = int(qm[1].zero_point.item()) - 128
    w1p = np.pad(w1, ((0, 0), (0, 0), (0, 0), (1, 1), (1, 1)), mode="reflect")
    w2 = Br.qconv3d(w1p, qm[2].weight_int8.numpy(), z1, np.float32(qm[1].scale.item()), qm[2].weight_scale.numpy(),
                    bias=qm[2].bias.numpy(), **req(qm[2]))
    assert np.array_equal(volume_codes(y2), w2)
    y3 = qm[3](y2)
    w3 = Br.qconv_transpose3d(w2, qm[3].weight_int8.numpy(), int(qm[2].zero_point.item()) - 128,
                              np.float32(qm[2].scale.item()), qm[3].weight_scale.numpy(), stride=(2, 2, 2),
                              bias=qm[3].bias.numpy(), **req(qm[3]))
    assert np.array_equal(volume_codes(y3), w3)
    out = qm(hip(x)).numpy()
    exp = (w3.astype(np.float32) + 128 - np.float32(qm[3].zero_point.item())) * np.float32(qm[3].scale.item())
    assert out.shape == (2, 8, 8, 12, 10) and np.array_equal(out, exp)
