"""GPU tests of the module layer: ``quantize_dynamic`` / ``convert`` install
hip int8 modules whose results are bit-exact against the oracle's integer
formulation and within tolerance of Lucid's float pass structure.

The structure follows the reference's own suites
(lucid/test/unit/quantization/test_dynamic_ptq.py, test_static_ptq.py,
test_functional_module.py, test_real_gemm.py:148-157)."""

import warnings

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.backends as backends
import lucid_amd.nn as nn
import lucid_amd.nn.intrinsic as nni
import lucid_amd.nn.quantized as nnq
import lucid_amd.nn.quantized.dynamic as nnqd
import lucid_amd.quantization as Q
import oracle as O

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


def _set(linear, w, b):
    linear.register_buffer("weight", L.tensor(w))
    linear.register_buffer("bias", L.tensor(b))


def _mlp(rng, sizes=(784, 256, 10), std=0.05):
    layers, params = [], []
    for i in range(len(sizes) - 1):
        lin = nn.Linear(sizes[i], sizes[i + 1])
        w = (rng.standard_normal((sizes[i + 1], sizes[i])) * std).astype(np.float32)
        b = (rng.standard_normal(sizes[i + 1]) * std).astype(np.float32)
        _set(lin, w, b)
        params.append((w, b))
        layers.append(lin)
        if i < len(sizes) - 2:
            layers.append(nn.ReLU())
    return nn.Sequential(*layers), params


def _oracle_weight(w):
    mn, mx = O.minmax(w, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    return O.quantize(w, ws, wz, -128, 127, ch_axis=0), ws, wz


def _oracle_dynamic_linear(x, w, b):
    """nnqd.Linear (dynamic/linear.py:84-99) in the integer formulation, plus
    the reference's float pass structure for the tolerance check."""
    wq, ws, wz = _oracle_weight(w)
    mn, mx = O.minmax(x)
    xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
    xq = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
    y_int = O.qlinear(xq, wq, int(xz[0]) - 128, xs, ws, bias=b, out_mode=O.OUT_F32)
    y_float = O.linear_faithful(O.fake_quantize(x, xs, xz, 0, 255), wq, ws, wz, bias=b)
    return y_int, y_float


# ------------------------------------------------------------------ dynamic PTQ
class TestDynamicPTQ:
    def test_swaps_linear_and_keeps_int8_weight(self):
        # test_dynamic_ptq.py:34-38
        model, _ = _mlp(np.random.default_rng(0), (32, 64, 64, 10))
        qm = Q.quantize_dynamic(model)
        assert isinstance(qm[0], nnqd.Linear) and isinstance(qm[2], nnqd.Linear)
        assert isinstance(model[0], nn.Linear)          # not in place
        assert qm[0].weight_int8.dtype is L.int8 and qm[0].weight_int8.shape == (64, 32)
        assert qm[0].act_qdtype is Q.quint8

    def test_mlp_config_bit_exact_and_within_tolerance(self):
        """Linear(784,256)-ReLU-Linear(256,10), batch 64, seeded."""
        rng = np.random.default_rng(1)
        model, params = _mlp(rng)
        x = rng.standard_normal((64, 784)).astype(np.float32)
        qm = Q.quantize_dynamic(model)
        y = qm(hip(x))
        assert y.shape == (64, 10) and y.dtype is L.float32 and y._grid is None

        (w1, b1), (w2, b2) = params
        h_int, h_float = _oracle_dynamic_linear(x, w1, b1)
        h_int, h_float = np.maximum(h_int, 0), np.maximum(h_float, 0)
        y_int, _ = _oracle_dynamic_linear(h_int, w2, b2)
        _, y_float = _oracle_dynamic_linear(h_float, w2, b2)
        # every stage is bit-exact against the integer formulation
        wq1, ws1, _ = _oracle_weight(w1)
        assert np.array_equal(qm[0].weight_int8.numpy(), wq1)
        assert np.array_equal(qm[0].weight_scale.numpy(), ws1)
        h = qm[1](qm[0](hip(x)))
        assert np.array_equal(h.numpy().view(np.uint32), h_int.view(np.uint32))
        assert np.array_equal(y.numpy().view(np.uint32), y_int.view(np.uint32))
        # and within 1e-3 relative of the reference's float pass structure
        assert np.abs(y.numpy() - y_float).max() <= 1e-3 * np.abs(y_float).max()
        # quality bound of the reference's own test (test_dynamic_ptq.py:40-46)
        y_fp = np.maximum(x @ w1.T + b1, 0) @ w2.T + b2
        assert np.abs(y.numpy() - y_fp).mean() / np.abs(y_fp).mean() < 0.05

    def test_leading_dims_are_flattened(self):
        rng = np.random.default_rng(2)
        lin = nn.Linear(48, 24)
        w = (rng.standard_normal((24, 48)) * 0.1).astype(np.float32)
        b = rng.standard_normal(24).astype(np.float32)
        _set(lin, w, b)
        q = nnqd.Linear.from_float(lin)
        x = rng.standard_normal((3, 5, 48)).astype(np.float32)
        y = q(hip(x))
        assert y.shape == (3, 5, 24)
        y_int, _ = _oracle_dynamic_linear(x.reshape(15, 48), w, b)
        assert np.array_equal(y.numpy().reshape(15, 24).view(np.uint32), y_int.view(np.uint32))

    def test_no_target_warns(self):
        with pytest.warns(UserWarning, match="no module of a targeted type"):
            Q.quantize_dynamic(nn.Sequential(nn.ReLU()))

    def test_state_dict_round_trip_is_bit_equal(self):
        # test_static_ptq.py:132-145 (checkpoint round trip)
        rng = np.random.default_rng(3)
        model, _ = _mlp(rng, (64, 32, 8))
        qa, qb = Q.quantize_dynamic(model), Q.quantize_dynamic(_mlp(np.random.default_rng(9), (64, 32, 8))[0])
        sd = qa.state_dict()
        assert set(sd) == {"0.weight_int8", "0.weight_scale", "0.weight_zero_point", "0.bias",
                           "2.weight_int8", "2.weight_scale", "2.weight_zero_point", "2.bias"}
        host = {k: L.tensor(v.numpy()) for k, v in sd.items()}      # as if loaded from disk
        qb.load_state_dict({k: v.to("hip") for k, v in host.items()})
        x = hip(rng.standard_normal((16, 64)).astype(np.float32))
        assert np.array_equal(qa(x).numpy().view(np.uint32), qb(x).numpy().view(np.uint32))


# ------------------------------------------------------------------ static PTQ
def _static_model(rng):
    class MLP(nn.Module):
        def __init__(self):
            super().__init__()
            self.quant = nnq.QuantStub()
            self.fc1 = nni.LinearReLU(nn.Linear(16, 32), nn.ReLU())
            self.fc2 = nn.Linear(32, 8)
            self.dequant = nnq.DeQuantStub()

        def forward(self, x):
            return self.dequant(self.fc2(self.fc1(self.quant(x))))

    m = MLP()
    w1 = (rng.standard_normal((32, 16)) * 0.3).astype(np.float32)
    b1 = (rng.standard_normal(32) * 0.1).astype(np.float32)
    w2 = (rng.standard_normal((8, 32)) * 0.3).astype(np.float32)
    b2 = (rng.standard_normal(8) * 0.1).astype(np.float32)
    _set(m.fc1[0], w1, b1)
    _set(m.fc2, w2, b2)
    return m, (w1, b1, w2, b2)


def _calibrate(prepared, params, rng, batches=20):
    """Feeds the observers what a float forward of the model would show them
    (the float forward itself is Lucid's CPU / Metal job)."""
    w1, b1, w2, b2 = params
    for _ in range(batches):
        x = rng.standard_normal((64, 16)).astype(np.float32)
        h = np.maximum(x @ w1.T + b1, 0)
        y = h @ w2.T + b2
        prepared.quant.activation_post_process(hip(x))
        prepared.fc1.activation_post_process(hip(h))
        prepared.fc2.activation_post_process(hip(y))


class TestStaticPTQ:
    def test_convert_structure_and_numerics(self):
        rng = np.random.default_rng(0)
        m, params = _static_model(rng)
        prepared = Q.prepare(m, Q.get_default_qconfig())
        _calibrate(prepared, params, rng)
        qm = Q.convert(prepared)
        # test_static_ptq.py:66-76
        assert isinstance(qm.fc1, nnq.LinearReLU) and isinstance(qm.fc2, nnq.Linear)
        assert isinstance(qm.quant, nnq.Quantize) and isinstance(qm.dequant, nnq.DeQuantize)
        assert qm.fc1.weight_int8.dtype is L.int8 and qm.fc2.weight_int8.dtype is L.int8
        assert qm.fc1.out_qdtype is Q.quint8 and qm.fc1.scale.shape == ()

        w1, b1, w2, b2 = params
        x = rng.standard_normal((64, 16)).astype(np.float32)
        y = qm(hip(x))
        assert y._grid is None and y.dtype is L.float32

        # oracle, integer formulation, stage by stage
        s0, z0 = qm.quant.scale.item(), qm.quant.zero_point.item()
        s1, z1 = qm.fc1.scale.item(), qm.fc1.zero_point.item()
        s2, z2 = qm.fc2.scale.item(), qm.fc2.zero_point.item()
        xq = O.quantize(x, s0, z0, 0, 255, code_offset=-128)
        wq1, ws1, wz1 = _oracle_weight(w1)
        wq2, ws2, wz2 = _oracle_weight(w2)
        h = O.qlinear(xq, wq1, int(z0) - 128, s0, ws1, bias=b1, relu=True,
                      out_mode=O.OUT_REQUANT_I8, out_scale=s1, out_zp=z1, out_offset=-128)
        yq = O.qlinear(h, wq2, int(z1) - 128, s1, ws2, bias=b2, out_mode=O.OUT_REQUANT_I8,
                       out_scale=s2, out_zp=z2, out_offset=-128)
        inner = qm.fc2(qm.fc1(qm.quant(hip(x))))
        assert np.array_equal(inner._grid.codes.numpy(), yq)
        assert np.array_equal(y.numpy().view(np.uint32),
                              O.dequantize(yq, s2, z2, code_offset=-128).view(np.uint32))

        # Lucid's float pass structure: codes agree up to +-1 on rounding ties
        xf = O.fake_quantize(x, s0, z0, 0, 255)
        hf = O.linear_faithful(xf, wq1, ws1, wz1, bias=b1, relu=True, fq=(s1, z1, 0, 255))
        yf = O.linear_faithful(hf, wq2, ws2, wz2, bias=b2, fq=(s2, z2, 0, 255))
        assert np.abs(y.numpy() - yf).max() <= s2 * 1.001
        assert (y.numpy() != yf).mean() < 0.02
        # quality bound of the reference's own test (test_static_ptq.py:78-86)
        y_fp = np.maximum(x @ w1.T + b1, 0) @ w2.T + b2
        assert np.abs(y.numpy() - y_fp).mean() / np.abs(y_fp).mean() < 0.05

    @pytest.mark.parametrize("ext", ["lucid", "safetensors"])
    def test_checkpoint_file_round_trip_is_bit_equal(self, tmp_path, ext):
        """test_static_ptq.py:132-145: save(state_dict) -> load -> load_state_dict into a
        freshly calibrated twin gives the same output bits, and int8 stays int8."""
        rng = np.random.default_rng(0)
        m, params = _static_model(rng)
        prepared = Q.prepare(m, Q.get_default_qconfig())
        _calibrate(prepared, params, rng)
        qm = Q.convert(prepared)
        x = hip(rng.standard_normal((64, 16)).astype(np.float32))
        before = qm(x).numpy()
        path = str(tmp_path / f"qmodel.{ext}")
        if ext == "lucid":
            L.save(qm.state_dict(), path)
        else:
            L.serialization.save_safetensors(qm.state_dict(), path)
        loaded = L.load(path)
        assert loaded["fc1.weight_int8"].dtype is L.int8 and loaded["fc1.weight_int8"].device == "cpu"
        assert loaded["fc1.scale"].shape == ()
        rng2 = np.random.default_rng(77)  # a twin with other weights and another calibration
        m2, params2 = _static_model(rng2)
        prepared2 = Q.prepare(m2, Q.get_default_qconfig())
        _calibrate(prepared2, params2, rng2)
        qm2 = Q.convert(prepared2)
        assert not np.array_equal(qm2(x).numpy(), before)
        qm2.load_state_dict(loaded)
        assert qm2.fc1.weight_int8.device == "hip"
        assert np.array_equal(qm2(x).numpy().view(np.uint32), before.view(np.uint32))

    def test_uncalibrated_convert_warns(self):
        # lucid/test/unit/quantization/test_safety.py (warning text "never saw")
        m, _ = _static_model(np.random.default_rng(1))
        prepared = Q.prepare(m)
        with pytest.warns(UserWarning, match="never saw"):
            Q.convert(prepared)

    def test_prepare_without_targets_warns(self):
        with pytest.warns(UserWarning, match="matched no quantizable"):
            Q.prepare(nn.Sequential(nn.ReLU()))

    def test_plain_float_input_runs_lucids_float_formulation(self):
        """A float input that lies on no grid takes Lucid's own path
        (linear.py:199-215): dequantized weight, float GEMM, fake-quantized output."""
        rng = np.random.default_rng(2)
        m, params = _static_model(rng)
        prepared = Q.prepare(m)
        _calibrate(prepared, params, rng, batches=2)
        qm = Q.convert(prepared)
        x = rng.standard_normal((9, 16)).astype(np.float32)
        y = qm.fc1(hip(x))
        assert y._grid is None and y.shape == (9, 32)
        wq1, ws1, wz1 = _oracle_weight(params[0])
        s1, z1 = qm.fc1.scale.item(), qm.fc1.zero_point.item()
        ref = O.linear_faithful(x, wq1, ws1, wz1, bias=params[1], relu=True, fq=(s1, z1, 0, 255))
        assert np.abs(y.numpy() - ref).max() <= s1 * 1.001 and (y.numpy() != ref).mean() < 0.02
        with pytest.raises(L.DeviceMismatch):
            qm(L.tensor(np.zeros((4, 16), np.float32)))

    def test_quantize_passes_integer_inputs_through(self):
        # lucid/test/unit/quantization/test_breadth.py:38-46
        q = nnq.Quantize(hip(np.float32(0.1)), hip(np.float32(0.0)))
        idx = hip(np.arange(6, dtype=np.int64))
        assert q(idx) is idx


# ------------------------------------------------------------------ affine weights
def _affine_qconfig():
    from lucid_amd.quantization.observer import HistogramObserver, PerChannelMinMaxObserver
    return Q.QConfig(activation=HistogramObserver.with_args(qscheme=Q.per_tensor_affine, qdtype=Q.quint8),
                     weight=PerChannelMinMaxObserver.with_args(ch_axis=0, qscheme=Q.per_channel_affine,
                                                               qdtype=Q.qint8))


def _oracle_affine_weight(w):
    mn, mx = O.minmax(w, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, False, -128, 127, True)
    return O.quantize(w, ws, wz, -128, 127, ch_axis=0), ws, wz


def test_static_ptq_with_per_channel_affine_weights():
    """A weight observer with qscheme per_channel_affine gives non-zero weight zero points;
    convert() keeps them and the int8 forward applies them: bit-exact against the oracle's
    integer formulation, within a code of Lucid's float composite."""
    rng = np.random.default_rng(4)
    m, params = _static_model(rng)
    w1, b1, w2, b2 = params
    w1 = (w1 + rng.uniform(-0.5, 0.5, (32, 1))).astype(np.float32)   # rows off centre: zero points != 0
    w2 = (w2 + rng.uniform(-0.5, 0.5, (8, 1))).astype(np.float32)
    _set(m.fc1[0], w1, b1)
    _set(m.fc2, w2, b2)
    params = (w1, b1, w2, b2)
    prepared = Q.prepare(m, _affine_qconfig())
    _calibrate(prepared, params, rng)
    qm = Q.convert(prepared)
    assert np.any(qm.fc1.weight_zero_point.numpy() != 0) and np.any(qm.fc2.weight_zero_point.numpy() != 0)
    x = rng.standard_normal((64, 16)).astype(np.float32)
    y = qm(hip(x)).numpy()
    s0, z0 = qm.quant.scale.item(), qm.quant.zero_point.item()
    s1, z1 = qm.fc1.scale.item(), qm.fc1.zero_point.item()
    s2, z2 = qm.fc2.scale.item(), qm.fc2.zero_point.item()
    xq = O.quantize(x, s0, z0, 0, 255, code_offset=-128)
    wq1, ws1, wz1 = _oracle_affine_weight(w1)
    wq2, ws2, wz2 = _oracle_affine_weight(w2)
    assert np.array_equal(qm.fc1.weight_int8.numpy(), wq1) and np.array_equal(qm.fc1.weight_zero_point.numpy(), wz1)
    h = O.qlinear(xq, wq1, int(z0) - 128, s0, ws1, bias=b1, relu=True, out_mode=O.OUT_REQUANT_I8,
                  out_scale=s1, out_zp=z1, out_offset=-128, w_zp=wz1.astype(np.int32))
    yq = O.qlinear(h, wq2, int(z1) - 128, s1, ws2, bias=b2, out_mode=O.OUT_REQUANT_I8,
                   out_scale=s2, out_zp=z2, out_offset=-128, w_zp=wz2.astype(np.int32))
    assert np.array_equal(y.view(np.uint32), O.dequantize(yq, s2, z2, code_offset=-128).view(np.uint32))
    xf = O.fake_quantize(x, s0, z0, 0, 255)
    hf = O.linear_faithful(xf, wq1, ws1, wz1, bias=b1, relu=True, fq=(s1, z1, 0, 255))
    yf = O.linear_faithful(hf, wq2, ws2, wz2, bias=b2, fq=(s2, z2, 0, 255))
    assert np.abs(y - yf).max() <= s2 * 1.001 and (y != yf).mean() < 0.02
    # a state_dict round trip keeps the zero points in force
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")  # the twin is converted uncalibrated on purpose
        qm2 = Q.convert(Q.prepare(_static_model(np.random.default_rng(9))[0], _affine_qconfig()))
    qm2.load_state_dict(qm.state_dict())
    assert np.array_equal(qm2(hip(x)).numpy().view(np.uint32), y.view(np.uint32))


def test_dynamic_linear_with_affine_weights():
    rng = np.random.default_rng(6)
    lin = nnqd.Linear(48, 24)
    w = codes = rng.integers(-128, 128, (24, 48)).astype(np.int8)
    zw = rng.integers(-60, 60, 24).astype(np.float32)
    ws = rng.uniform(0.001, 0.004, 24).astype(np.float32)
    b = rng.standard_normal(24).astype(np.float32)
    lin.load_state_dict({"weight_int8": L.tensor(w), "weight_scale": L.tensor(ws), "weight_zero_point": L.tensor(zw),
                         "bias": L.tensor(b)})
    x = rng.standard_normal((10, 48)).astype(np.float32)
    y = lin(hip(x)).numpy()
    mn, mx = O.minmax(x)
    xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
    xq = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
    exp = O.qlinear(xq, codes, int(xz[0]) - 128, xs, ws, bias=b, w_zp=zw.astype(np.int32))
    assert np.array_equal(y.view(np.uint32), exp.view(np.uint32))
    with pytest.raises(ValueError, match="int8 codes"):
        lin.load_state_dict({"weight_int8": L.tensor(w), "weight_scale": L.tensor(ws),
                             "weight_zero_point": L.tensor(zw + 0.5), "bias": L.tensor(b)})
        lin(hip(x))


# ------------------------------------------------------------------ residual join
def test_qfunctional_add_relu_matches_oracle():
    rng = np.random.default_rng(5)
    a = (rng.standard_normal((4, 500)) * 2).astype(np.float32)
    b = (rng.standard_normal((4, 500)) * 3).astype(np.float32)
    qa = nnq.Quantize(hip(np.float32(0.05)), hip(np.float32(120.0)))
    qb = nnq.Quantize(hip(np.float32(0.07)), hip(np.float32(131.0)))
    f = nnq.QFunctional(hip(np.float32(0.06)), hip(np.float32(0.0)))
    out = f.add_relu(qa(hip(a)), qb(hip(b)))
    ca = O.quantize(a, 0.05, 120.0, 0, 255, code_offset=-128)
    cb = O.quantize(b, 0.07, 131.0, 0, 255, code_offset=-128)
    exp = O.add_requant(ca, -128, np.float32(0.05), 120.0, cb, -128, np.float32(0.07), 131.0, True,
                        np.float32(0.06), 0.0, 0, 255, -128)
    assert np.array_equal(out._grid.codes.numpy(), exp)
    # float view equals Lucid's composition fq(relu(x + y)) on the float-carried operands
    xa, xb = O.fake_quantize(a, 0.05, 120.0, 0, 255), O.fake_quantize(b, 0.07, 131.0, 0, 255)
    ref = O.fake_quantize(np.maximum(xa + xb, 0), 0.06, 0.0, 0, 255)
    assert np.array_equal(out.numpy().view(np.uint32), ref.view(np.uint32))
    out2 = nnq.QFunctional(hip(np.float32(0.06)), hip(np.float32(128.0))).add(qa(hip(a)), qb(hip(b)))
    ref2 = O.fake_quantize(xa + xb, 0.06, 128.0, 0, 255)
    assert np.array_equal(out2.numpy().view(np.uint32), ref2.view(np.uint32))


def test_qfunctional_mul_scalars_and_cat_match_the_float_composition():
    """functional_module.py:220-246: each merge is fake_quantize(op(x, y)) on
    float-carried operands; on codes it must give the same bits."""
    rng = np.random.default_rng(6)
    a = (rng.standard_normal((4, 300)) * 2).astype(np.float32)
    b = (rng.standard_normal((4, 300)) * 3).astype(np.float32)
    qa = nnq.Quantize(hip(np.float32(0.05)), hip(np.float32(120.0)))
    qb = nnq.Quantize(hip(np.float32(0.07)), hip(np.float32(131.0)))
    xa, xb = O.fake_quantize(a, 0.05, 120.0, 0, 255), O.fake_quantize(b, 0.07, 131.0, 0, 255)
    f = nnq.QFunctional(hip(np.float32(0.11)), hip(np.float32(125.0)))
    same = lambda got, ref: np.array_equal(got.numpy().view(np.uint32), ref.view(np.uint32))
    assert same(f.mul(qa(hip(a)), qb(hip(b))), O.fake_quantize(xa * xb, 0.11, 125.0, 0, 255))
    assert same(f.add_scalar(qa(hip(a)), 0.3), O.fake_quantize(xa + np.float32(0.3), 0.11, 125.0, 0, 255))
    assert same(f.mul_scalar(qa(hip(a)), -1.7), O.fake_quantize(xa * np.float32(-1.7), 0.11, 125.0, 0, 255))
    got = f.cat([qa(hip(a)), qb(hip(b))], dim=1)
    assert got.shape == (4, 600)
    assert same(got, O.fake_quantize(np.concatenate([xa, xb], 1), 0.11, 125.0, 0, 255))
    got0 = f.cat([qa(hip(a)), qb(hip(b))], dim=0)
    assert got0.shape == (8, 300)
    assert same(got0, O.fake_quantize(np.concatenate([xa, xb], 0), 0.11, 125.0, 0, 255))
    # channel concatenation of 4-d activations (stored NHWC)
    u = (rng.standard_normal((2, 5, 6, 7)) * 2).astype(np.float32)
    v = (rng.standard_normal((2, 9, 6, 7)) * 2).astype(np.float32)
    xu, xv = O.fake_quantize(u, 0.05, 120.0, 0, 255), O.fake_quantize(v, 0.07, 131.0, 0, 255)
    got4 = f.cat([qa(hip(u)), qb(hip(v))], dim=1)
    assert got4.shape == (2, 14, 6, 7)
    assert same(got4, O.fake_quantize(np.concatenate([xu, xv], 1), 0.11, 125.0, 0, 255))


def test_observers_known_answers_on_device():
    # lucid/test/unit/quantization/test_observer.py:12-17,43-50
    obs = Q.MinMaxObserver()
    obs(hip([[-1.0, 2.0], [0.5, 3.0]]))
    obs(hip([[-2.0, 1.0]]))
    assert obs.min_val.item() == -2.0 and obs.max_val.item() == 3.0
    scale, zp = obs.calculate_qparams()
    assert scale.item() == pytest.approx(5.0 / 255.0, rel=1e-5) and 0 <= zp.item() <= 255
    pc = Q.PerChannelMinMaxObserver(ch_axis=0)
    pc(hip([[1.0, 2.0, 3.0], [-4.0, 0.5, 0.1]]))
    assert pc.min_val.numpy().tolist() == [1.0, -4.0] and pc.max_val.numpy().tolist() == [3.0, 0.5]
    s, z = pc.calculate_qparams()
    assert s.shape == (2,) and z.numpy().tolist() == [0.0, 0.0]
    pc(hip([[5.0, -9.0, 0.0], [0.0, 0.0, 7.0]]))
    assert pc.min_val.numpy().tolist() == [-9.0, -4.0] and pc.max_val.numpy().tolist() == [5.0, 7.0]
    fx = Q.FixedQParamsObserver(1.0 / 256, 0)
    assert fx.calculate_qparams()[0].item() == 1.0 / 256


def test_relu_kernel():
    x = np.array([-1.0, -0.0, 0.0, 2.5, np.nan, -np.inf, np.inf] * 37, np.float32)
    y = nn.relu(hip(x)).numpy()
    exp = np.where(x < 0, np.float32(0), x)
    assert np.array_equal(y.view(np.uint32)[~np.isnan(x)], exp.view(np.uint32)[~np.isnan(x)])
    assert np.isnan(y[np.isnan(x)]).all()


def test_engine_toggle():
    # lucid/test/unit/quantization/test_real_gemm.py:148-157
    prev = backends.quantized.engine
    try:
        for v in ("auto", "reference", "mlx_group", "hip"):
            backends.quantized.engine = v
            assert backends.quantized.engine == v
        with pytest.raises(ValueError):
            backends.quantized.engine = "cuda"
        backends.quantized.engine = "hip"
        assert backends.quantized.available and backends.quantized.use_hip()
        assert not backends.quantized.use_mlx()
    finally:
        backends.quantized.engine = prev


@pytest.mark.parametrize("M,K,N", [(64, 784, 256), (64, 256, 10), (1, 16, 1), (17, 48, 33), (5, 1024, 70), (64, 1024, 16),
                                   (33, 1040, 100), (3, 6080, 40)])
@pytest.mark.parametrize("kind", ["normal", "constant", "nan"])
def test_small_dynamic_linear_in_one_launch(M, K, N, kind):
    """lq_dynamic_linear_small_f32 (min / max, qparams, codes, GEMM and bias of nnqd.Linear in one
    launch) gives the bits of lq_quantize_tensor_dynamic_i8 followed by lq_qlinear_i8, and of the
    oracle's integer formulation, on ragged shapes, a constant input (scale at eps) and a NaN."""
    from lucid_amd import _C, _ops
    rng = np.random.default_rng(M * 3 + K + N)
    x = rng.standard_normal((M, K)).astype(np.float32) * 3
    if kind == "constant":
        x[:] = 0.0
    elif kind == "nan":
        x[M // 2, K // 3] = np.nan
    w = rng.integers(-127, 128, (N, K)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, N).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    xd, wd, wsd, bd = hip(x), hip(w), hip(ws), hip(b)
    wsum = _ops.rowsum_i8(wd)
    for relu, bias in ((0, bd), (1, bd), (0, None)):
        y = L.Tensor.empty((M, N), L.float32, "hip")
        _C.call("lq_dynamic_linear_small_f32", xd.data_ptr, M, K, wd.data_ptr, N, wsd.data_ptr, wsum.data_ptr,
                None if bias is None else bias.data_ptr, relu, 0, 0, 255, 0, 1e-8, -128, y.data_ptr, None)
        xq = L.Tensor.empty((M, K), L.int8, "hip")
        s, z = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
        _C.call("lq_quantize_tensor_dynamic_i8", xd.data_ptr, M * K, 0, 0, 255, 0, 1e-8, -128, s.data_ptr, z.data_ptr,
                None, None, xq.data_ptr, None)
        two = _ops.qlinear_i8(xq, wd, a_zp=-128, a_zp_dev=z, a_scale=s, w_scale=wsd, wsum=wsum, bias=bias,
                              relu=bool(relu), out_mode=_ops.OUT_F32)
        got, want = y.numpy(), two.numpy()
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(got[~np.isnan(got)].view(np.uint32), want[~np.isnan(want)].view(np.uint32))
        if kind == "normal" and relu == 0 and bias is not None:
            mn, mx = O.minmax(x)
            xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
            codes = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
            exp = O.qlinear(codes, w, int(xz[0]) - 128, xs, ws, bias=b, out_mode=O.OUT_F32)
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))
    with pytest.raises(NotImplementedError, match="up to 64 rows"):
        _C.call("lq_dynamic_linear_small_f32", xd.data_ptr, 65, K, wd.data_ptr, N, wsd.data_ptr, wsum.data_ptr, None, 0, 0,
                0, 255, 0, 1e-8, -128, y.data_ptr, None)


@pytest.mark.parametrize("K", [6080, 6096, 8192, 11008, 16384])
@pytest.mark.parametrize("M", [1, 4])
def test_dynamic_linear_wide_layer_at_small_batch(M, K):
    """nnqd.Linear on a layer too wide for the one-launch kernel (16 K bytes of codes must fit
    96 KiB of LDS: K <= 6080) takes the two-launch route at any batch size, with the bits the
    one-launch kernel would give: checked against the explicit quantize + GEMM pair."""
    import lucid_amd.nn.quantized.dynamic as nnqd
    from lucid_amd import _C, _ops
    from lucid_amd.nn.quantized.dynamic.linear import SMALL_LINEAR_MAX_K
    rng = np.random.default_rng(K + M)
    N = 48
    lin = nnqd.Linear(K, N)
    w = rng.integers(-127, 128, (N, K)).astype(np.int8)
    lin.weight_int8 = hip(w)
    lin.weight_scale = hip(rng.uniform(0.001, 0.01, N).astype(np.float32))
    lin.bias = hip(rng.standard_normal(N).astype(np.float32))
    lin._state_loaded("weight_int8")
    x = (rng.standard_normal((M, K)) * 2).astype(np.float32)
    xd = hip(x)
    y = lin(xd).numpy()
    xq = L.Tensor.empty((M, K), L.int8, "hip")
    s, z = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
    _C.call("lq_quantize_tensor_dynamic_i8", xd.data_ptr, M * K, 0, 0, 255, 0, 1e-8, -128, s.data_ptr, z.data_ptr,
            None, None, xq.data_ptr, None)
    want = _ops.qlinear_i8(xq, lin.weight_int8, a_zp=-128, a_zp_dev=z, a_scale=s, w_scale=lin.weight_scale,
                           wsum=_ops.rowsum_i8(lin.weight_int8), bias=lin.bias, out_mode=_ops.OUT_F32).numpy()
    assert y.shape == (M, N)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    if K > SMALL_LINEAR_MAX_K:
        out = L.Tensor.empty((M, N), L.float32, "hip")
        with pytest.raises(NotImplementedError, match="K <= 6080"):
            _C.call("lq_dynamic_linear_small_f32", xd.data_ptr, M, K, lin.weight_int8.data_ptr, N,
                    lin.weight_scale.data_ptr, _ops.rowsum_i8(lin.weight_int8).data_ptr, None, 0, 0, 0, 255, 0, 1e-8,
                    -128, out.data_ptr, None)


class _recorded_calls:
    """The names of the compute entry points called through the binding while the block runs."""

    def __enter__(self):
        from lucid_amd import _C
        self._C, self._orig, self.names = _C, _C.call, []

        def call(name, *args):
            if name not in ("lq_alloc", "lq_free", "lq_sync", "lq_d2h", "lq_h2d", "lq_rowsum_i8"):  # one-off weight prep
                self.names.append(name)
            return self._orig(name, *args)

        _C.call = call
        return self.names

    def __exit__(self, *exc):
        self._C.call = self._orig
        return False


@pytest.mark.parametrize("M,K1,N1,N2", [(64, 784, 256, 10), (5, 64, 16, 1), (33, 1024, 240, 64), (17, 48, 32, 10)])
@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("kind", ["normal", "constant", "nan"])
def test_two_dynamic_linears_in_one_launch(M, K1, N1, N2, relu, kind):
    """A Sequential of nnqd.Linear [, ReLU], nnqd.Linear on a small batch runs as ONE launch
    (lq_dynamic_mlp2_small_f32: the last block of layer 1 to finish reduces the hidden activation's
    min / max and runs layer 2): bit for bit what the modules give one after the other, and what
    the oracle's integer formulation gives."""
    rng = np.random.default_rng(M + K1 + N1 + N2)
    l1, l2 = nn.Linear(K1, N1), nn.Linear(N1, N2)
    l1.register_buffer("weight", L.tensor((rng.standard_normal((N1, K1)) * 0.05).astype(np.float32)))
    l1.register_buffer("bias", L.tensor((rng.standard_normal(N1) * 0.05).astype(np.float32)))
    l2.register_buffer("weight", L.tensor((rng.standard_normal((N2, N1)) * 0.05).astype(np.float32)))
    l2.register_buffer("bias", L.tensor((rng.standard_normal(N2) * 0.05).astype(np.float32)))
    mods = [l1, nn.ReLU(), l2] if relu else [l1, l2]
    model = Q.quantize_dynamic(nn.Sequential(*mods))
    x = rng.standard_normal((M, K1)).astype(np.float32)
    if kind == "constant":
        x[:] = 0.25
    elif kind == "nan":
        x[M // 2, K1 // 3] = np.nan
    xd = hip(x)
    with _recorded_calls() as calls:
        got_t = model(xd)
    assert calls == ["lq_dynamic_mlp2_small_f32"]        # one kernel launch for the whole model
    got = got_t.numpy()
    h = model[0](xd)
    if relu:
        h = model[1](h)
    want = model[-1](h).numpy()
    assert got.shape == (M, N2)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)].view(np.uint32), want[~np.isnan(want)].view(np.uint32))
    if kind == "normal":
        q1, q2 = model[0], model[-1]
        mn, mx = O.minmax(x)
        xs, xz = O.calc_qparams(mn, mx, False, 0, 255, False)
        c1 = O.quantize(x, xs, xz, 0, 255, code_offset=-128)
        hh = O.qlinear(c1, q1.weight_int8.numpy(), int(xz[0]) - 128, xs, q1.weight_scale.numpy(), bias=q1.bias.numpy(),
                       relu=relu, out_mode=O.OUT_F32)
        mn, mx = O.minmax(hh)
        hs, hz = O.calc_qparams(mn, mx, False, 0, 255, False)
        c2 = O.quantize(hh, hs, hz, 0, 255, code_offset=-128)
        exp = O.qlinear(c2, q2.weight_int8.numpy(), int(hz[0]) - 128, hs, q2.weight_scale.numpy(), bias=q2.bias.numpy(),
                        out_mode=O.OUT_F32)
        assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))


def test_two_dynamic_linears_keep_separate_launches_when_hooked_or_large():
    """A forward hook has to see each module's own output, and a wide layer is not what the one
    launch takes: the modules then run one after the other."""
    rng = np.random.default_rng(3)
    model = Q.quantize_dynamic(nn.Sequential(nn.Linear(64, 32), nn.ReLU(), nn.Linear(32, 8)))
    x = hip(rng.standard_normal((4, 64)).astype(np.float32))
    seen = []
    model[0].register_forward_hook(lambda mod, inp, out: seen.append(out.shape))
    y = model(x)
    assert seen == [(4, 32)] and y.shape == (4, 8)
    big = Q.quantize_dynamic(nn.Sequential(nn.Linear(64, 512), nn.Linear(512, 8)))
    with _recorded_calls() as calls:
        assert big(x).shape == (4, 8)
    assert "lq_dynamic_mlp2_small_f32" not in calls and len(calls) >= 2


def test_two_dynamic_linears_are_captured_as_separate_launches_with_the_same_bits():
    """Under graph capture the pair is not fused (the two layers' own kernels are shorter than the
    one launch, which only saves the host a launch); the replayed result equals the eager, fused
    one bit for bit - also with fused launches on other inputs between the replays."""
    rng = np.random.default_rng(5)
    model = Q.quantize_dynamic(nn.Sequential(nn.Linear(784, 256), nn.ReLU(), nn.Linear(256, 10)))
    x = hip(rng.standard_normal((64, 784)).astype(np.float32))
    with _recorded_calls() as calls:
        eager = model(x).numpy()
    assert calls == ["lq_dynamic_mlp2_small_f32"]
    with L.graph.capture() as g:
        with _recorded_calls() as calls:
            y = model(x)
    assert "lq_dynamic_mlp2_small_f32" not in calls and calls.count("lq_dynamic_linear_small_f32") == 2
    other = hip(rng.standard_normal((7, 784)).astype(np.float32) * 3)
    other_eager = model[2](model[1](model[0](other))).numpy()
    for _ in range(3):
        g.replay()
        L.synchronize()
        assert np.array_equal(y.numpy().view(np.uint32), eager.view(np.uint32))
        # the one launch again, smaller: its arrival counter and scratch are the previous call's
        assert np.array_equal(model(other).numpy().view(np.uint32), other_eager.view(np.uint32))
    g.destroy()
