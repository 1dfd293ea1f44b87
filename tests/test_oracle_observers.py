"""Calibration-side observers of the oracle against the reference's own tests and
independent implementations; CPU only."""

import random

import numpy as np
import pytest
import torch

import oracle as O
import oracle.observers as OB


def test_histc_against_numpy_histogram():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(50000).astype(np.float32)
    lo, hi = float(x.min()), float(x.max())
    got = OB.histc(x, 256, lo, hi)
    ref, _ = np.histogram(x.astype(np.float64), bins=256, range=(lo, hi))
    # numpy places a value on an inner edge by comparison with the edge array, the
    # reference by truncating (v - lo) / step: they may differ on edge values only
    assert got.sum() == 50000 and np.abs(got - ref).sum() <= 4
    # right edge into the last bin, outside values skipped (CpuBackend.h:13306-13310)
    h = OB.histc(np.array([0.0, 1.0, 2.0, 3.0, -1.0, 5.0], np.float32), 3, 0.0, 3.0)
    assert h.tolist() == [1.0, 1.0, 2.0]


def test_moving_average_known_answer():
    # test_observer.py:34-39: c = 0.5, [-2, 2] then [-4, 4] -> (-3, 3)
    mn = OB.ema(np.float32(np.inf), np.float32(-2.0), 0.5, True)
    mx = OB.ema(np.float32(-np.inf), np.float32(2.0), 0.5, True)
    mn = OB.ema(mn, np.float32(-4.0), 0.5, False)
    mx = OB.ema(mx, np.float32(4.0), 0.5, False)
    assert mn == -3.0 and mx == 3.0


def test_moving_average_against_torch_observer():
    # test_observer_parity.py:60-74: c = 0.1, four batches of default_rng(2)
    rng = np.random.default_rng(2)
    tobs = torch.ao.quantization.MovingAverageMinMaxObserver(averaging_constant=0.1, dtype=torch.quint8)
    mn, mx, first = np.float32(np.inf), np.float32(-np.inf), True
    for _ in range(4):
        x = rng.standard_normal((4, 8)).astype(np.float32)
        tobs(torch.from_numpy(x))
        mn, mx = OB.ema(mn, x.min(), 0.1, first), OB.ema(mx, x.max(), 0.1, first)
        first = False
    assert float(mn) == pytest.approx(float(tobs.min_val), abs=1e-6)
    assert float(mx) == pytest.approx(float(tobs.max_val), abs=1e-6)
    s, z = O.calc_qparams(mn, mx, False, 0, 255, False)
    ts, tz = tobs.calculate_qparams()
    assert float(s[0]) == pytest.approx(float(ts), abs=1e-6) and abs(float(z[0]) - float(tz)) <= 1


def test_histogram_observer_reference_properties():
    # test_observer.py:53-62
    random.seed(0)
    obs = OB.HistogramObserver(bins=256)
    obs(np.array([random.gauss(0.0, 1.0) for _ in range(2000)], np.float32))
    assert obs.histogram.sum() == pytest.approx(2000, abs=2)
    assert obs.qparams()[0] > 0.0
    # test_observer.py:64-76: the L2 clip range is no wider than raw min / max
    random.seed(1)
    data = np.array([random.gauss(0.0, 1.0) for _ in range(3000)] +
                    [random.uniform(5.0, 12.0) for _ in range(150)], np.float32)
    h = OB.HistogramObserver(bins=512)
    h(data)
    s_mm, _ = O.calc_qparams(data.min(), data.max(), False, 0, 255, False)
    assert h.qparams()[0] <= s_mm[0]
    lo, hi = h.clip_range()
    assert lo >= float(data.min()) and hi <= float(data.max()) and hi < 12.0  # the tail was clipped


def test_histogram_rebinning_conserves_mass_and_matches_a_fresh_histogram():
    rng = np.random.default_rng(3)
    a = rng.standard_normal(20000).astype(np.float32)
    b = (rng.standard_normal(20000) * 3).astype(np.float32)  # wider: forces a re-bin
    obs = OB.HistogramObserver(bins=128)
    obs(a)
    obs(b)
    assert obs.histogram.sum() == 40000
    both = np.concatenate([a, b])
    fresh = OB.histc(both, 128, obs.min_val, obs.max_val)
    # re-binning moves a whole old bin to the new bin of its centre: close to, not equal to, a fresh count
    assert np.abs(obs.histogram - fresh).sum() / 40000 < 0.05
