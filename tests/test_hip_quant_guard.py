"""The quantize kernels replace x / s by a guarded reciprocal multiply.  These
tests aim at the guard: operands on and next to rounding ties, quotients that
the reciprocal would round to the other side, extreme scales, and a dense
sweep of float32 bit patterns - all must equal the IEEE-division oracle."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.quantization as Q
import oracle as O

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


@pytest.mark.parametrize("s", [0.1, 0.037, 1.0 / 3.0, 0.05, 4.0 / 255.0, 0.02, 0.017, 1e-8, 3.0,
                               1.1754944e-38, 6e-39, 1e30, 0.4699588716030121])
def test_near_tie_operands(s):
    s = np.float32(s)
    n = np.arange(-300, 301, dtype=np.float64)
    base = ((n + 0.5) * np.float64(s)).astype(np.float32)     # nearest float to each tie
    xs = [base]
    for k in (1, 2, 3, 5):
        xs.append(np.nextafter(xs[-1], np.float32(np.inf)))
    lo = base
    for k in range(4):
        lo = np.nextafter(lo, np.float32(-np.inf))
        xs.append(lo)
    x = np.concatenate(xs)
    x = np.concatenate([x, np.zeros((-x.size) % 1024, np.float32)])
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        exp = O.quantize(x, s, 7.0, -128, 127)
    assert np.array_equal(Q.quantize(hip(x), float(s), 7.0, Q.qint8).numpy(), exp)
    exp_fq = O.fake_quantize(x, s, 7.0, -128, 127)
    got_fq = Q.fake_quantize(hip(x), float(s), 7.0, -128, 127).numpy()
    ok = (got_fq.view(np.uint32) == exp_fq.view(np.uint32)) | (np.isnan(got_fq) & np.isnan(exp_fq))
    assert ok.all()


@pytest.mark.parametrize("seed", range(3))
def test_dense_bit_pattern_sweep(seed):
    """2^22 float32 bit patterns (all exponents, random mantissas) x 8 scales."""
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 2 ** 32, 1 << 22, dtype=np.uint64).astype(np.uint32)
    x = bits.view(np.float32).copy()
    x[np.isnan(x)] = 0.0
    for s in rng.uniform(1e-3, 0.5, 4).astype(np.float32).tolist() + [1e-20, 1e20, 2.0 ** -10, 7.0]:
        s = np.float32(s)
        with np.errstate(over="ignore", invalid="ignore"):
            exp = O.quantize(x, s, 128.0, 0, 255, q_dtype=O.I16)
        got = Q.quantize(hip(x), float(s), 128.0, Q.quint8).numpy()
        assert np.array_equal(got, exp), f"scale {s}"


def test_scaled_normal_data_many_scales():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((64, 4096)) * rng.uniform(0.01, 100, (64, 1))).astype(np.float32)
    mn, mx = O.minmax(x, ch_axis=0)
    s, z = O.calc_qparams(mn, mx, True, -128, 127, True)
    got = Q.quantize(hip(x), hip(s), hip(z), Q.qint8, ch_axis=0).numpy()
    assert np.array_equal(got, O.quantize(x, s, z, -128, 127, ch_axis=0))


@pytest.mark.parametrize("relu", [0, 1])
@pytest.mark.parametrize("scale,zp,qmin,qmax", [
    (0.05, 0.0, -128, 127), (0.037, 128.0, 0, 255), (1.0, -5.0, -128, 127), (0.5, 3.0, 0, 255),
    (3.0, 0.0, -128, 127), (0.1, 64.0, 0, 255), (7.3e-4, 17.0, 0, 255), (0.0314, 64.0, 0, 255),
    (1e-30, 0.0, -128, 127), (1e30, 0.0, -128, 127), (0.02, 300.0, 0, 255), (-0.25, 0.0, -128, 127),
    (0.04, -3.0, 0, 255), (0.04, 200.0, -128, 127), (0.04, 0.5, -128, 127), (0.04, 255.0, 0, 255),
    (0.04, -128.0, -128, 127)])
def test_tile_epilogue_requantize_route_on_every_float32(scale, zp, qmin, qmax, relu):
    """The GEMM / convolution epilogue requantizes through a reciprocal multiply where that is
    provably the same and divides elsewhere; a ReLU directly before it is folded into the lower
    clamp bound, and a fused join takes the code minus its zero point from shifted bounds.
    Every one of the 2^32 float32 bit patterns (all finite values, both zeros, subnormals,
    infinities, every NaN) must give, in both forms, the code that the plain [floor at zero,]
    divide-round-add-clamp gives.  A tiny or huge scale, a zero point beyond 255 or not an
    integer are outside what the reciprocal route accepts, and under a ReLU so are a negative
    scale and a zero point outside the code range: there every pattern must take the dividing
    branch (without a ReLU a negative scale is accepted like a positive one)."""
    from lucid_amd import _C
    bad = L.Tensor.empty((1,), L.int64, "hip")
    slow = L.Tensor.empty((1,), L.int64, "hip")
    _C.call("lq_selftest_requant_route", scale, zp, qmin, qmax, relu, 0, 1 << 32, bad.data_ptr, slow.data_ptr, None)
    assert int(bad.numpy()[0]) == 0
    divided = int(slow.numpy()[0])
    refused = abs(scale) < 1e-20 or abs(scale) > 1e20 or abs(zp) > 255 or zp != round(zp)
    if relu:
        refused = refused or scale < 0 or not (qmin <= zp <= qmax)
    if refused:
        assert divided == 1 << 32
    else:
        # NaNs, infinities and the huge-quotient tail always divide; of the rest only a sliver
        assert (1 << 24) < divided < (1 << 32) // 20


def test_tile_epilogue_requantize_route_random_grids():
    """The same exhaustive comparison on 48 random grids (scales log-uniform in 1e-5..1e2,
    integer zero points, both code ranges, with and without the folded ReLU)."""
    from lucid_amd import _C
    rng = np.random.default_rng(2024)
    bad = L.Tensor.empty((1,), L.int64, "hip")
    slow = L.Tensor.empty((1,), L.int64, "hip")
    for i in range(48):
        scale = float(np.float32(10.0 ** rng.uniform(-5, 2)))
        signed = bool(i % 2)
        qmin, qmax = (-128, 127) if signed else (0, 255)
        zp = float(rng.integers(qmin, qmax + 1))
        relu = (i // 2) % 2
        _C.call("lq_selftest_requant_route", scale, zp, qmin, qmax, relu, 0, 1 << 32, bad.data_ptr, slow.data_ptr,
                None)
        assert int(bad.numpy()[0]) == 0, (scale, zp, qmin, qmax, relu)
