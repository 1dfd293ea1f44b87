"""prepare -> calibrate -> convert -> infer entirely on the device
(lucid/test/unit/quantization/test_device_metal.py is the template: the same recipe,
with "hip" in place of "metal" and a numpy float model in place of the CPU run)."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.quantization as Q

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.asarray(a, np.float32), device="hip")


def _static_quant(qconfig):
    rng = np.random.default_rng(0)
    m = nn.Sequential(nn.Linear(16, 16), nn.ReLU(), nn.Linear(16, 8)).to("hip")
    qm = Q.prepare(m, qconfig)
    for _ in range(4):
        qm(hip(rng.standard_normal((4, 16))))       # observers are fed by the float forward
    cm = Q.convert(qm)
    x = np.array([[0.1 * i - 0.8 for i in range(16)] for _ in range(4)], np.float32)
    w0, b0, w2, b2 = (t.numpy() for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias))
    return cm, cm(hip(x)), np.maximum(x @ w0.T + b0, 0) @ w2.T + b2


def test_float_linear_forward_matches_numpy():
    rng = np.random.default_rng(1)
    lin = nn.Linear(48, 24).to("hip")
    x = rng.standard_normal((5, 7, 48)).astype(np.float32)
    y = lin(hip(x)).numpy()
    want = x @ lin.weight.numpy().T + lin.bias.numpy()
    assert y.shape == (5, 7, 24) and np.abs(y - want).max() < 1e-5


def test_static_ptq_round_trip_on_device():
    # test_device_metal.py:53-65: no crash, finite, and within quantization noise of the float model
    cm, y, yf = _static_quant(Q.get_default_qconfig())
    assert y.device == "hip"
    out = y.numpy()
    assert np.isfinite(out).all()
    assert np.abs(out - yf).max() < 5e-2


def test_qat_qconfig_static_quant_on_device():
    # test_device_metal.py:65-68: the FakeQuantize-based qconfig through the same static flow
    cm, y, yf = _static_quant(Q.get_default_qat_qconfig())
    out = y.numpy()
    assert np.isfinite(out).all() and np.abs(out - yf).max() < 1e-1


def test_observers_were_fed_by_the_forward_hooks():
    rng = np.random.default_rng(2)
    m = nn.Sequential(nn.Linear(16, 16), nn.ReLU(), nn.Linear(16, 8)).to("hip")
    qm = Q.prepare(m, Q.QConfig(activation=Q.MinMaxObserver, weight=Q.get_default_qconfig().weight))
    xs = [rng.standard_normal((4, 16)).astype(np.float32) for _ in range(3)]
    for x in xs:
        qm(hip(x))
    w0, b0 = m[0].weight.numpy(), m[0].bias.numpy()
    h = np.concatenate([x @ w0.T + b0 for x in xs])
    obs = qm[0].activation_post_process
    assert np.isclose(obs.min_val.numpy(), h.min(), atol=1e-5) and np.isclose(obs.max_val.numpy(), h.max(), atol=1e-5)


@pytest.mark.parametrize("factory", [Q.MinMaxObserver, Q.MovingAverageMinMaxObserver,
                                     lambda: Q.PerChannelMinMaxObserver(ch_axis=0),
                                     lambda: Q.MovingAveragePerChannelMinMaxObserver(ch_axis=0),
                                     Q.HistogramObserver])
def test_observers_calibrate_on_device(factory):
    # test_device_metal.py:75-95
    obs = factory()
    x = np.random.default_rng(3).standard_normal((4, 8)).astype(np.float32)
    obs(hip(x))
    obs(hip(x * 1.5))
    scale, zero_point = obs.calculate_qparams()
    assert np.isfinite(scale.numpy()).all() and np.isfinite(zero_point.numpy()).all()


def test_fake_quantize_takes_cpu_qparams_on_a_device_input():
    # test_device_metal.py:98-109
    x = hip(np.random.default_rng(4).standard_normal((4, 8)))
    out = Q.fake_quantize(x, L.tensor(np.float32(0.05)), L.tensor(np.float32(0.0)), -128, 127, None)
    assert out.device == "hip" and np.isfinite(out.numpy()).all()


def _conv2d_numpy(x, w, b, stride, pad, dil, groups):
    B, C, H, W = x.shape
    O, Cg, KH, KW = w.shape
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (pad[0], pad[0]), (pad[1], pad[1])))
    OH = (H + 2 * pad[0] - dil[0] * (KH - 1) - 1) // stride[0] + 1
    OW = (W + 2 * pad[1] - dil[1] * (KW - 1) - 1) // stride[1] + 1
    out = np.zeros((B, O, OH, OW))
    og = O // groups
    for o in range(O):
        g = o // og
        for kh in range(KH):
            for kw in range(KW):
                sl = xp[:, g * Cg:(g + 1) * Cg, kh * dil[0]:kh * dil[0] + (OH - 1) * stride[0] + 1:stride[0],
                        kw * dil[1]:kw * dil[1] + (OW - 1) * stride[1] + 1:stride[1]]
                out[:, o] += np.tensordot(sl, w[o, :, kh, kw].astype(np.float64), axes=([1], [0]))
        if b is not None:
            out[:, o] += b[o]
    return out


@pytest.mark.parametrize("cin,cout,k,stride,pad,dil,groups,hw", [
    (3, 16, 7, 2, 3, 1, 1, (30, 29)), (16, 32, 3, 1, 1, 1, 1, (14, 14)), (32, 32, (3, 1), (2, 1), (1, 0), (1, 2), 4, (9, 11)),
    (8, 24, 1, 1, 0, 1, 1, (5, 5)), (16, 16, 3, 1, 2, 2, 16, (12, 12))])
def test_float_conv2d_forward_matches_numpy(cin, cout, k, stride, pad, dil, groups, hw):
    pair = lambda v: (v, v) if isinstance(v, int) else v
    rng = np.random.default_rng(cin + cout)
    conv = nn.Conv2d(cin, cout, k, stride=stride, padding=pad, dilation=dil, groups=groups).to("hip")
    x = rng.standard_normal((2, cin, *hw)).astype(np.float32)
    y = conv(hip(x)).numpy()
    want = _conv2d_numpy(x, conv.weight.numpy(), conv.bias.numpy(), pair(stride), pair(pad), pair(dil), groups)
    assert y.shape == want.shape
    assert np.abs(y - want).max() <= 1e-4 * (1 + np.abs(want).max())


def test_conv_model_calibrates_and_converts_on_device():
    """prepare -> calibrate (float convolutions on the device feed the observers) -> convert -> infer
    for a small convolutional model, against its float forward."""
    import lucid_amd.nn.quantized as nnq
    rng = np.random.default_rng(5)
    import lucid_amd.nn.intrinsic as nni
    m = nn.Sequential(nnq.QuantStub(), nni.ConvReLU2d(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU()),
                      nn.Conv2d(32, 16, 1), nnq.DeQuantStub()).to("hip")
    qm = Q.prepare(m, Q.get_default_qconfig())
    for _ in range(4):
        qm(hip(rng.standard_normal((2, 16, 12, 12))))
    cm = Q.convert(qm)
    assert isinstance(cm[1], nnq.ConvReLU2d) and isinstance(cm[2], nnq.Conv2d)
    x = rng.standard_normal((2, 16, 12, 12)).astype(np.float32)
    yf = m(hip(x)).numpy()
    yq = cm(hip(x)).numpy()
    assert yq.shape == yf.shape and np.isfinite(yq).all()
    assert np.abs(yq - yf).mean() / np.abs(yf).mean() < 0.05
