"""The inference side of quantization-aware training on the hip device: ``prepare_qat``
installs ``nn.qat`` layers whose forward fake-quantizes weights and outputs
(``lucid/nn/qat/linear.py``, ``lucid/quantization/_fake_quantize.py``), and ``convert`` bakes
them into the int8 modules.  Forward only; compared with the oracle's fake-quantize and
float linear, and with the converted int8 model."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.nn.qat as nnqat
import lucid_amd.nn.quantized as nnq
import lucid_amd.nn.intrinsic as nni
import lucid_amd.quantization as Q
import oracle as O

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


def _model():
    return nn.Sequential(nnq.QuantStub(), nni.LinearReLU(nn.Linear(48, 32), nn.ReLU()), nn.Linear(32, 10),
                         nnq.DeQuantStub())


def test_default_qat_qconfig_builds_fake_quantize_pairs():
    qc = Q.get_default_qat_qconfig()
    a, w = qc.activation(), qc.weight()
    assert type(a).__name__ == "FakeQuantize" and type(w).__name__ == "FakeQuantize"
    assert a.qdtype is Q.quint8 and a.ch_axis is None and w.qdtype is Q.qint8 and w.ch_axis == 0
    assert type(a.activation_post_process).__name__ == "MovingAverageMinMaxObserver"
    assert type(w.activation_post_process).__name__ == "PerChannelMinMaxObserver"


def test_fake_quantize_module_observes_then_transforms():
    rng = np.random.default_rng(0)
    fq = Q.FakeQuantize(observer=Q.MinMaxObserver, qscheme=Q.per_tensor_affine, qdtype=Q.quint8)
    x = rng.standard_normal((5, 40)).astype(np.float32) * 3
    y = fq(hip(x)).numpy()
    s, z = O.calc_qparams(np.float32(x.min()), np.float32(x.max()), False, 0, 255, False)
    assert np.array_equal(fq.scale.numpy().ravel().view(np.uint32), np.asarray(s, np.float32).ravel().view(np.uint32))
    assert np.array_equal(y.view(np.uint32), O.fake_quantize(x, s, z, 0, 255).view(np.uint32))
    fq.disable_observer()
    x2 = x * 10
    y2 = fq(hip(x2)).numpy()          # frozen qparams: saturates instead of widening
    assert np.array_equal(y2.view(np.uint32), O.fake_quantize(x2, s, z, 0, 255).view(np.uint32))
    fq.disable_fake_quant()
    assert np.array_equal(fq(hip(x2)).numpy(), x2)


def test_prepare_qat_forward_and_convert():
    rng = np.random.default_rng(1)
    qat = Q.prepare_qat(_model())
    assert isinstance(qat[1], nnqat.LinearReLU) and isinstance(qat[2], nnqat.Linear)
    assert type(qat[0].activation_post_process).__name__ == "FakeQuantize"
    for _ in range(5):                      # the moving averages settle on the data
        y = qat(hip(rng.standard_normal((16, 48)).astype(np.float32)))
    # freeze the statistics, then check the forward against the composition it stands for
    for m in qat.modules():
        if type(m).__name__ == "FakeQuantize":
            m.disable_observer()
    x = rng.standard_normal((16, 48)).astype(np.float32)
    y = qat(hip(x)).numpy()

    def fq(t, m, ch_axis=None):
        return O.fake_quantize(t, m.scale.numpy(), m.zero_point.numpy(), m.qdtype.quant_min, m.qdtype.quant_max,
                               ch_axis=ch_axis)

    h = fq(x, qat[0].activation_post_process)
    l1, l2 = qat[1], qat[2]
    w1 = fq(l1.weight.numpy(), l1.weight_fake_quant, 0)
    h = np.maximum(h @ w1.T + l1.bias.numpy(), 0).astype(np.float32)
    h = fq(h, l1.activation_post_process)
    w2 = fq(l2.weight.numpy(), l2.weight_fake_quant, 0)
    ref = fq((h @ w2.T + l2.bias.numpy()).astype(np.float32), l2.activation_post_process)
    step = float(l2.activation_post_process.scale.numpy())
    d = np.abs(y - ref)
    assert d.max() <= step * 1.001 and (d > step * 0.01).mean() < 0.02   # float GEMM order: rare one-step flips
    # convert: int8 modules with the QAT qparams; same function within a quantization step
    q8 = Q.convert(qat)
    assert isinstance(q8[1], nnq.LinearReLU) and isinstance(q8[2], nnq.Linear) and isinstance(q8[0], nnq.Quantize)
    assert q8[2].weight_int8.dtype is L.int8
    assert np.array_equal(q8[2].weight_scale.numpy().ravel().view(np.uint32),
                          l2.weight_fake_quant.scale.numpy().ravel().view(np.uint32))
    y8 = q8(hip(x)).numpy()
    d8 = np.abs(y8 - y)
    assert d8.max() <= step * 2.001 and (d8 > step * 0.01).mean() < 0.05


def test_prepare_qat_convolutional_model_forward_and_convert():
    rng = np.random.default_rng(3)
    m = nn.Sequential(nnq.QuantStub(), nni.ConvReLU2d(nn.Conv2d(16, 32, 3, padding=1), nn.ReLU()),
                      nn.Conv2d(32, 16, 1), nnq.DeQuantStub())
    qat = Q.prepare_qat(m)
    assert isinstance(qat[1], nnqat.ConvReLU2d) and isinstance(qat[2], nnqat.Conv2d)
    for _ in range(5):
        qat(hip(rng.standard_normal((2, 16, 10, 10)).astype(np.float32)))
    for mod in qat.modules():
        if type(mod).__name__ == "FakeQuantize":
            mod.disable_observer()
    x = rng.standard_normal((2, 16, 10, 10)).astype(np.float32)
    y = qat(hip(x)).numpy()
    # the forward is the float convolution of fake-quantized operands, fake-quantized
    c1 = qat[1]
    fq = lambda t, mm, ax=None: O.fake_quantize(t, mm.scale.numpy(), mm.zero_point.numpy(), mm.qdtype.quant_min,
                                                mm.qdtype.quant_max, ch_axis=ax)
    h = fq(x, qat[0].activation_post_process)
    conv = nn.Conv2d(16, 32, 3, padding=1)
    conv.register_buffer("weight", hip(fq(c1.weight.numpy(), c1.weight_fake_quant, 0)))
    conv.register_buffer("bias", c1.bias)
    h1 = fq(np.maximum(conv(hip(h)).numpy(), 0), c1.activation_post_process)
    step1 = float(c1.activation_post_process.scale.numpy())
    got1 = qat[1](qat[0](hip(x))).numpy()
    assert np.abs(got1 - h1).max() <= step1 * 1.001
    q8 = Q.convert(qat)
    assert isinstance(q8[1], nnq.ConvReLU2d) and isinstance(q8[2], nnq.Conv2d)
    y8 = q8(hip(x)).numpy()
    step = float(qat[2].activation_post_process.scale.numpy())
    d = np.abs(y8 - y)
    assert d.max() <= step * 2.001 and (d > step * 0.01).mean() < 0.05
