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


def _fq(t, mm, ax=None):
    return O.fake_quantize(t, mm.scale.numpy(), mm.zero_point.numpy(), mm.qdtype.quant_min, mm.qdtype.quant_max,
                           ch_axis=ax)


def _freeze(model):
    for mod in model.modules():
        if type(mod).__name__ == "FakeQuantize":
            mod.disable_observer()


@pytest.mark.parametrize("rank", [1, 3])
def test_prepare_qat_in_one_and_three_dimensions(rank):
    """nn.qat.Conv1d / Conv3d and their ConvReLU forms (lucid/nn/qat/conv.py:46,328,476,697):
    prepare_qat installs them, the forward is the float convolution of fake-quantized operands,
    convert bakes them into the int8 modules of the same rank."""
    rng = np.random.default_rng(rank)
    if rank == 1:
        shape = (2, 16, 40)
        m = nn.Sequential(nnq.QuantStub(), nni.ConvReLU1d(nn.Conv1d(16, 32, 3, padding=1), nn.ReLU()),
                          nn.Conv1d(32, 16, 1), nnq.DeQuantStub())
        kinds = (nnqat.ConvReLU1d, nnqat.Conv1d, nnq.ConvReLU1d, nnq.Conv1d)
    else:
        shape = (2, 16, 4, 6, 6)
        m = nn.Sequential(nnq.QuantStub(), nni.ConvReLU3d(nn.Conv3d(16, 32, 3, padding=1), nn.ReLU()),
                          nn.Conv3d(32, 16, 1), nnq.DeQuantStub())
        kinds = (nnqat.ConvReLU3d, nnqat.Conv3d, nnq.ConvReLU3d, nnq.Conv3d)
    qat = Q.prepare_qat(m)
    assert isinstance(qat[1], kinds[0]) and isinstance(qat[2], kinds[1])
    for _ in range(5):
        qat(hip(rng.standard_normal(shape).astype(np.float32)))
    _freeze(qat)
    x = rng.standard_normal(shape).astype(np.float32)
    y = qat(hip(x)).numpy()
    c1 = qat[1]
    h = _fq(x, qat[0].activation_post_process)
    conv = (nn.Conv1d if rank == 1 else nn.Conv3d)(16, 32, 3, padding=1)
    conv.register_buffer("weight", hip(_fq(c1.weight.numpy(), c1.weight_fake_quant, 0)))
    conv.register_buffer("bias", c1.bias)
    h1 = _fq(np.maximum(conv(hip(h)).numpy(), 0), c1.activation_post_process)
    got1 = qat[1](qat[0](hip(x))).numpy()
    assert np.abs(got1 - h1).max() <= float(c1.activation_post_process.scale.numpy()) * 1.001
    q8 = Q.convert(qat)
    assert isinstance(q8[1], kinds[2]) and isinstance(q8[2], kinds[3])
    y8 = q8(hip(x)).numpy()
    step = float(qat[2].activation_post_process.scale.numpy())
    d = np.abs(y8 - y)
    assert d.max() <= step * 2.001 and (d > step * 0.01).mean() < 0.05


def test_float_conv3d_forward_matches_torch():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(7)
    for cin, cout, k, stride, pad, dil, groups, shape in [(4, 6, 3, 1, 1, 1, 1, (2, 4, 5, 6, 7)),
                                                           (6, 8, (1, 3, 2), (1, 2, 1), (0, 1, 1), (1, 1, 2), 2, (1, 6, 3, 9, 8))]:
        conv = nn.Conv3d(cin, cout, k, stride=stride, padding=pad, dilation=dil, groups=groups)
        x = rng.standard_normal(shape).astype(np.float32)
        y = conv(hip(x)).numpy()
        ref = torch.nn.functional.conv3d(torch.from_numpy(x), torch.from_numpy(conv.weight.numpy()),
                                         torch.from_numpy(conv.bias.numpy()), stride, pad, dil, groups).numpy()
        assert y.shape == ref.shape and np.abs(y - ref).max() <= 2e-5 * max(1.0, np.abs(ref).max())


def test_qat_embedding_forward_and_convert():
    """nn.qat.Embedding (lucid/nn/qat/sparse.py:21): the looked-up rows are rows of the
    fake-quantized table; convert bakes the table into nnq.Embedding with the same qparams."""
    rng = np.random.default_rng(5)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.emb = nn.Embedding(50, 12, padding_idx=0)

        def forward(self, idx):
            return self.emb(idx)

    net = Net()
    qat = Q.prepare_qat(net)
    assert isinstance(qat.emb, nnqat.Embedding) and not hasattr(qat.emb, "activation_post_process")
    idx = rng.integers(0, 50, (4, 9)).astype(np.int64)
    got = qat(hip(idx)).numpy()
    wfq = qat.emb.weight_fake_quant
    table = _fq(qat.emb.weight.numpy(), wfq, 0)
    assert got.shape == (4, 9, 12) and np.array_equal(got.view(np.uint32), table[idx].view(np.uint32))
    q8 = Q.convert(qat)
    assert isinstance(q8.emb, nnq.Embedding) and q8.emb.weight_int8.dtype is L.int8
    assert np.array_equal(q8(hip(idx)).numpy().view(np.uint32), got.view(np.uint32))
    with pytest.raises(ValueError, match="qconfig"):
        nnqat.Embedding(5, 3)


@pytest.mark.parametrize("rank,relu", [(1, False), (2, True), (3, True)])
def test_fuse_modules_qat_conv_bn_forward_and_convert(rank, relu):
    """nn.intrinsic.qat.ConvBn* / ConvBnReLU* (lucid/nn/intrinsic/qat/modules.py:30-860):
    fuse_modules_qat builds them, the forward folds the BatchNorm into the weight before
    fake-quantizing it, convert bakes the folded weight into the int8 convolution."""
    import lucid_amd.nn.intrinsic.qat as nniqat
    from lucid_amd.nn.utils import fuse_conv_bn_eval
    rng = np.random.default_rng(10 + rank)
    conv_cls = (nn.Conv1d, nn.Conv2d, nn.Conv3d)[rank - 1]
    bn_cls = (nn.BatchNorm1d, nn.BatchNorm2d, nn.BatchNorm3d)[rank - 1]
    shape = [(2, 8, 30), (2, 8, 9, 9), (2, 8, 3, 5, 5)][rank - 1]

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.quant = nnq.QuantStub()
            self.conv = conv_cls(8, 16, 3, padding=1)
            self.bn = bn_cls(16)
            self.relu = nn.ReLU()
            self.dequant = nnq.DeQuantStub()

        def forward(self, x):
            return self.dequant(self.relu(self.bn(self.conv(self.quant(x)))))

    net = Net().eval()
    n = 16
    net.bn.register_buffer("weight", L.tensor(rng.uniform(0.5, 1.5, n).astype(np.float32)))
    net.bn.register_buffer("bias", L.tensor(rng.standard_normal(n).astype(np.float32) * 0.2))
    net.bn.register_buffer("running_mean", L.tensor(rng.standard_normal(n).astype(np.float32) * 0.2))
    net.bn.register_buffer("running_var", L.tensor(rng.uniform(0.5, 2.0, n).astype(np.float32)))
    qconfig = Q.get_default_qat_qconfig()
    group = ["conv", "bn", "relu"] if relu else ["conv", "bn"]
    fused = Q.fuse_modules_qat(net, [group], qconfig)
    want = ((nniqat.ConvBn1d, nniqat.ConvBn2d, nniqat.ConvBn3d),
            (nniqat.ConvBnReLU1d, nniqat.ConvBnReLU2d, nniqat.ConvBnReLU3d))[int(relu)][rank - 1]
    assert type(fused.conv) is want and isinstance(fused.bn, nn.Identity)
    qat = Q.prepare_qat(fused, qconfig)
    assert type(qat.conv) is want                       # already a QAT form: left alone
    for _ in range(5):
        qat(hip(rng.standard_normal(shape).astype(np.float32)))
    _freeze(qat)
    x = rng.standard_normal(shape).astype(np.float32)
    y = qat(hip(x)).numpy()
    # stage by stage: fake-quantized input, folded + fake-quantized weight, float conv, (ReLU,) fake-quantized
    cb = qat.conv
    folded = fuse_conv_bn_eval(net.conv, net.bn)
    ref_conv = conv_cls(8, 16, 3, padding=1)
    ref_conv.register_buffer("weight", hip(_fq(folded.weight.numpy(), cb.weight_fake_quant, 0)))
    ref_conv.register_buffer("bias", folded.bias.to("hip"))
    h = ref_conv(hip(_fq(x, qat.quant.activation_post_process))).numpy()
    if not relu:
        ref = np.maximum(_fq(h, cb.activation_post_process), 0)   # the model's own ReLU follows the fused pair
    else:
        ref = _fq(np.maximum(h, 0), cb.activation_post_process)
    step = float(cb.activation_post_process.scale.numpy())
    assert np.abs(y - ref).max() <= step * 1.001
    q8 = Q.convert(qat)
    kinds = ((nnq.Conv1d, nnq.Conv2d, nnq.Conv3d), (nnq.ConvReLU1d, nnq.ConvReLU2d, nnq.ConvReLU3d))[int(relu)]
    assert type(q8.conv) is kinds[rank - 1] and q8.conv.weight_int8.dtype is L.int8
    y8 = q8(hip(x)).numpy()
    d = np.abs(y8 - y)
    assert d.max() <= step * 2.001 and (d > step * 0.01).mean() < 0.05
    with pytest.raises(ValueError):
        Q.fuse_modules_qat(net, [["bn", "relu"]], qconfig)
