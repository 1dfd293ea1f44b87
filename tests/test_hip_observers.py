"""Calibration-side observers on the device against the CPU restatement
(oracle/observers.py) and the reference's own known answers."""

import random

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.quantization as Q
import oracle as O
import oracle.observers as OB
from lucid_amd import _C

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.asarray(a, np.float32), device="hip")


@pytest.mark.parametrize("n,bins", [(50000, 256), (1, 16), (1 << 20, 2048), (777, 3)])
def test_histc_counts_are_exact(n, bins):
    rng = np.random.default_rng(n + bins)
    x = (rng.standard_normal(n) * 2).astype(np.float32)
    lo, hi = float(x.min()) - 0.25, float(x.max())  # right edge included, some room on the left
    out = L.Tensor.empty((bins,), L.float32, "hip")
    _C.call("lq_histc_f32", hip(x).data_ptr, n, lo, hi, bins, out.data_ptr, None)
    assert np.array_equal(out.numpy(), OB.histc(x, bins, lo, hi))
    # values outside the range are skipped
    _C.call("lq_histc_f32", hip(x).data_ptr, n, -0.5, 0.5, bins, out.data_ptr, None)
    assert np.array_equal(out.numpy(), OB.histc(x, bins, -0.5, 0.5))
    with pytest.raises(ValueError):
        _C.call("lq_histc_f32", hip(x).data_ptr, n, 1.0, 1.0, bins, out.data_ptr, None)  # hi must be > lo


def test_moving_average_observers():
    # known answer, test_observer.py:34-39
    obs = Q.MovingAverageMinMaxObserver(averaging_constant=0.5)
    obs(hip([-2.0, 2.0]))
    obs(hip([-4.0, 4.0]))
    assert obs.min_val.item() == -3.0 and obs.max_val.item() == 3.0
    # a longer run against the restatement, bit for bit
    rng = np.random.default_rng(2)
    obs = Q.MovingAverageMinMaxObserver(averaging_constant=0.1)
    pc = Q.MovingAveragePerChannelMinMaxObserver(ch_axis=0, averaging_constant=0.1)
    mn, mx, first = np.float32(np.inf), np.float32(-np.inf), True
    cmn = cmx = None
    for _ in range(5):
        x = rng.standard_normal((6, 40)).astype(np.float32)
        obs(hip(x))
        pc(hip(x))
        mn, mx = OB.ema(mn, x.min(), 0.1, first), OB.ema(mx, x.max(), 0.1, first)
        cmn = x.min(1) if first else OB.ema(cmn, x.min(1), 0.1, False)
        cmx = x.max(1) if first else OB.ema(cmx, x.max(1), 0.1, False)
        first = False
    assert obs.min_val.numpy().tobytes() == np.float32(mn).tobytes()
    assert obs.max_val.numpy().tobytes() == np.float32(mx).tobytes()
    assert np.array_equal(pc.min_val.numpy(), cmn) and np.array_equal(pc.max_val.numpy(), cmx)
    s, z = pc.calculate_qparams()
    es, ez = O.calc_qparams(cmn, cmx, True, -128, 127, True)
    assert np.array_equal(s.numpy(), es) and np.array_equal(z.numpy(), ez)


def test_histogram_observer_matches_the_restatement_and_the_reference_properties():
    # test_observer.py:53-62
    random.seed(0)
    data = np.array([random.gauss(0.0, 1.0) for _ in range(2000)], np.float32)
    obs = Q.HistogramObserver(bins=256)
    obs(hip(data))
    assert obs.histogram.numpy().sum() == pytest.approx(2000, abs=2)
    scale, zp = obs.calculate_qparams()
    assert scale.item() > 0.0
    # test_observer.py:64-76
    random.seed(1)
    data = np.array([random.gauss(0.0, 1.0) for _ in range(3000)] +
                    [random.uniform(5.0, 12.0) for _ in range(150)], np.float32)
    h, m = Q.HistogramObserver(bins=512), Q.MinMaxObserver()
    h(hip(data))
    m(hip(data))
    assert h.calculate_qparams()[0].item() <= m.calculate_qparams()[0].item()

    # several batches of growing range: histogram, range and qparams equal the restatement's
    rng = np.random.default_rng(4)
    dev, ref = Q.HistogramObserver(bins=2048), OB.HistogramObserver(bins=2048)
    for k in range(4):
        x = (rng.standard_normal((32, 500)) * (1 + k)).astype(np.float32)
        dev(hip(x))
        ref(x)
        assert np.array_equal(dev.histogram.numpy(), ref.histogram), k
        assert dev.min_val.item() == ref.min_val and dev.max_val.item() == ref.max_val
    s, z = dev.calculate_qparams()
    es, ez = ref.qparams()
    assert s.numpy().tobytes() == np.float32(es).tobytes() and z.item() == ez


def test_default_qconfig_is_lucids():
    # test_observer.py:104-107
    qc = Q.get_default_qconfig()
    assert isinstance(qc.weight(), Q.PerChannelMinMaxObserver)
    assert isinstance(qc.activation(), Q.HistogramObserver)
