"""CPU restatement of Lucid's calibration-side observers (numpy / python floats).

TEST INFRASTRUCTURE ONLY, like the rest of ``oracle/``.

* ``histc``                ``lucid/_C/backend/cpu/CpuBackend.h:13276-13316`` (double arithmetic,
                           right edge folded into the last bin, outside values skipped)
* ``HistogramObserver``    ``lucid/quantization/observer.py:773-895`` (range growth, re-binning
                           onto the wider range in float32 tensor steps, L2 clip search in
                           python floats)
* ``ema``                  ``observer.py:490-506`` / ``:1000-1018``

Pinned by the reference's own observer tests (``test_observer.py:34-39,53-76``: the moving
average known answer, histogram mass, clip range no wider than min/max), by numpy's
``histogram`` and by torch's ``MovingAverageMinMaxObserver`` as
``test_observer_parity.py:60-74`` uses it.
"""

from __future__ import annotations

import numpy as np

import oracle as O


def histc(x, bins, lo, hi):
    v = np.asarray(x, np.float32).reshape(-1).astype(np.float64)
    step = (float(hi) - float(lo)) / float(bins)
    keep = ~((v < lo) | (v > hi))
    b = ((v[keep] - lo) / step).astype(np.int64)
    b[b >= bins] = bins - 1
    counts = np.zeros(bins, np.float64)
    np.add.at(counts, b, 1.0)
    return counts.astype(np.float32)


def ema(run, cur, c, seed):
    run, cur = np.asarray(run, np.float32), np.asarray(cur, np.float32)
    with np.errstate(invalid="ignore"):  # inf - inf on the seeded lane, discarded by the select
        avg = (run + np.float32(c) * (cur - run)).astype(np.float32)
    return np.where(seed, cur, avg).astype(np.float32)


class HistogramObserver:
    def __init__(self, bins=2048, qmin=0, qmax=255):
        self.bins, self.qmin, self.qmax = bins, qmin, qmax
        self.min_val, self.max_val = float("inf"), float("-inf")
        self.histogram = np.zeros(bins, np.float32)

    def _rebin(self, hist, old_min, old_max, new_min, new_max):
        bins, f32 = self.bins, np.float32
        old_width = (old_max - old_min) / bins
        new_width = (new_max - new_min) / bins
        centers = f32(old_min) + (np.arange(bins).astype(f32) + f32(0.5)) * f32(old_width)
        raw = np.clip((centers - f32(new_min)) / f32(new_width), f32(0.0), f32(bins - 1)).astype(f32)
        out = np.zeros(bins, f32)
        np.add.at(out, raw.astype(np.int64), hist.astype(f32))
        return out

    def __call__(self, x):
        x = np.asarray(x, np.float32)
        cur_min, cur_max = float(x.min()), float(x.max())
        if self.min_val == float("inf"):
            new_min, new_max = cur_min, cur_max
            hist = histc(x, self.bins, new_min, new_max)
        else:
            new_min, new_max = min(self.min_val, cur_min), max(self.max_val, cur_max)
            hist = histc(x, self.bins, new_min, new_max)
            if new_min == self.min_val and new_max == self.max_val:
                hist = (hist + self.histogram).astype(np.float32)
            else:
                hist = (hist + self._rebin(self.histogram, self.min_val, self.max_val, new_min, new_max)
                        ).astype(np.float32)
        # the running range is stored in float32 buffers
        self.min_val, self.max_val = float(np.float32(new_min)), float(np.float32(new_max))
        self.histogram = hist
        return x

    def clip_range(self):
        lo, hi = self.min_val, self.max_val
        counts = [float(v) for v in self.histogram.tolist()]
        total = sum(counts)
        if total <= 0.0 or hi <= lo:
            return lo, hi
        bins = self.bins
        width = (hi - lo) / bins
        centers = [lo + (i + 0.5) * width for i in range(bins)]
        levels = self.qmax - self.qmin

        def quantile(q):
            target, acc = q * total, 0.0
            for c, n in zip(centers, counts):
                acc += n
                if acc >= target:
                    return c
            return centers[-1]

        best_err, best = float("inf"), (lo, hi)
        for frac in (0.0, 1e-5, 1e-4, 1e-3, 5e-3, 1e-2):
            cmin, cmax = quantile(frac), quantile(1.0 - frac)
            if cmax <= cmin:
                continue
            step = (cmax - cmin) / max(levels, 1)
            err = 0.0
            for c, n in zip(centers, counts):
                if n == 0.0:
                    continue
                cc = cmin if c < cmin else (cmax if c > cmax else c)
                err += n * ((c - cc) ** 2 + (step * step) / 12.0)
            if err < best_err:
                best_err, best = err, (cmin, cmax)
        return best

    def qparams(self):
        lo, hi = self.clip_range()
        s, z = O.calc_qparams(np.float32(lo), np.float32(hi), False, self.qmin, self.qmax, False)
        return s[0], z[0]
