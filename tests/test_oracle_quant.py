"""Pins the CPU oracle's quantize / dequantize / fake_quantize / qparams /
min-max / f16 functions.

Sources of truth, none of which is the oracle's own formula retyped:
  * known answers held by the reference's tests and docstrings (cited inline,
    paths relative to the Lucid checkout);
  * brute-force enumeration of rounding ties;
  * numpy's float32 division / rint / float16 conversion (library routines);
  * torch's quantize_per_tensor as the reference's parity tests use it.
"""

import numpy as np
import pytest

import oracle as O

QINT8 = (-128, 127)
QUINT8 = (0, 255)


# ------------------------------------------------------------------ known answers
def test_saturation_known_answer():
    # lucid/test/unit/quantization/test_functional.py:44-48
    q = O.quantize([-1000.0, 1000.0], 0.1, 0.0, *QINT8)
    assert q.dtype == np.int8 and q.tolist() == [-128, 127]


def test_affine_zero_point_known_answer():
    # test_functional.py:50-54 ; quint8 codes live in int16 (_qscheme.py:242-245)
    q = O.quantize([0.0], 0.02, 128.0, *QUINT8, q_dtype=O.I16)
    assert q.dtype == np.int16 and q.tolist() == [128]


def test_docstring_example_saturates():
    # lucid/quantization/_functional.py:146-148
    assert O.quantize([100.0], 0.05, 0.0, *QINT8).tolist() == [127]


def test_round_trip_on_grid():
    # test_functional.py:35-42
    x = np.array([-1.0, -0.3, 0.0, 0.7, 2.0], np.float32)
    q = O.quantize(x, 0.05, 0.0, *QINT8)
    dq = O.dequantize(q, 0.05, 0.0)
    assert np.allclose(dq, x, atol=1e-6)


def test_fake_quantize_equals_dequant_of_quant():
    # test_functional.py:58-63
    x = np.array([-1.0, -0.31, 0.0, 0.72, 2.0], np.float32)
    fq = O.fake_quantize(x, 0.05, 0.0, *QINT8)
    dq = O.dequantize(O.quantize(x, 0.05, 0.0, *QINT8), 0.05, 0.0)
    assert np.allclose(fq, dq, atol=1e-6)
    assert np.array_equal(fq, dq)  # same arithmetic, so in fact bit-equal


def test_per_channel_round_trip_bound():
    # test_functional.py:85-95
    w = np.array([[1.0, 2.0, 3.0], [-4.0, 0.5, 0.1]], np.float32)
    s = np.array([0.03, 0.05], np.float32)
    z = np.zeros(2, np.float32)
    q = O.quantize(w, s, z, *QINT8, ch_axis=0)
    dq = O.dequantize(q, s, z, ch_axis=0)
    assert (np.abs(dq - w) <= np.array([[0.03 / 2], [0.05 / 2]]) + 1e-6).all()


# ------------------------------------------------------------------ ties, brute force
@pytest.mark.parametrize("s", [0.5, 0.25, 2.0 ** -7, 1.0, 4.0])
@pytest.mark.parametrize("z,grid", [(0.0, QINT8), (128.0, QUINT8), (3.0, QINT8), (17.0, QUINT8)])
def test_ties_round_half_even(s, z, grid):
    # x = (n + 1/2) * s is exact for power-of-two s, so x / s is exactly a tie.
    n = np.arange(-400, 401)
    x = ((n + 0.5) * s).astype(np.float32)
    assert np.array_equal(x.astype(np.float64), (n + 0.5) * s)
    half_even = np.where(n % 2 == 0, n, n + 1)  # n+0.5 -> the even neighbour
    expect = np.clip(half_even + int(z), grid[0], grid[1])
    got = O.quantize(x, s, z, *grid, q_dtype=O.I16)
    assert np.array_equal(got, expect)


def test_round_then_add_order_matters():
    # Lucid rounds x/s first and adds z afterwards (_functional.py:180); adding
    # z before rounding would turn the tie 0.5 -> 0 into 1.5 -> 2.
    got = O.quantize([0.5], 1.0, 1.0, *QUINT8, q_dtype=O.I16)
    assert got.tolist() == [1]


def test_division_not_reciprocal():
    # x / s must be a correctly rounded division; x * (1/s) lands on the other
    # side of a tie for tens of thousands of these operands.
    rng = np.random.default_rng(123)
    n_diff = 0
    for _ in range(8):
        s = np.float32(rng.uniform(0.01, 0.2))
        n = rng.integers(-127, 127, 100000)
        x = ((n + 0.5) * np.float64(s)).astype(np.float32)  # nearest f32 to a tie
        differ = np.rint(x / s) != np.rint(x * (np.float32(1.0) / s))
        n_diff += int(differ.sum())
        got = O.quantize(x, s, 0.0, -1000, 1000, q_dtype=O.I16)
        # independent truth: the float64 quotient of two f32 values, rounded to
        # f32, is the correctly rounded f32 quotient (53 >= 2*24 + 2 bits)
        truth = np.rint((x.astype(np.float64) / np.float64(s)).astype(np.float32))
        assert np.array_equal(got, truth.astype(np.int16))
    assert n_diff > 1000, "search produced no discriminating operands"


# ------------------------------------------------------------------ numpy closed form
@pytest.mark.parametrize("seed", range(4))
def test_matches_numpy_float32_pipeline(seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((7, 33, 5)).astype(np.float32) * 3
    x.flat[::17] *= 50  # saturating values
    for ch_axis, n in [(None, 1), (0, 7), (1, 33), (2, 5), (-1, 5)]:
        s = (rng.uniform(0.005, 0.08, n)).astype(np.float32)
        z = rng.integers(0, 255, n).astype(np.float32)
        shape = [1] * 3
        if ch_axis is not None:
            shape[ch_axis] = n
        sb, zb = s.reshape(shape), z.reshape(shape)
        expect_f = np.clip(np.rint(x / sb) + zb, np.float32(0), np.float32(255))
        got = O.quantize(x, s, z, *QUINT8, ch_axis=ch_axis, q_dtype=O.I16)
        assert np.array_equal(got, expect_f.astype(np.int16))
        dq = O.dequantize(got, s, z, ch_axis=ch_axis)
        assert np.array_equal(dq, (got.astype(np.float32) - zb) * sb)
        fq = O.fake_quantize(x, s, z, *QUINT8, ch_axis=ch_axis)
        assert np.array_equal(fq, (expect_f - zb) * sb)


def test_fused_equals_faithful_bitwise():
    rng = np.random.default_rng(7)
    x = rng.standard_normal((6, 40, 9)).astype(np.float32) * 4
    # adversarial: exact ties, huge, tiny, denormal, infinities, signed zeros
    x.flat[:12] = [0.5 * 0.0625, 1.5 * 0.0625, -2.5 * 0.0625, 1e30, -1e30, 1e-42, -1e-42,
                   np.inf, -np.inf, 0.0, -0.0, 127.5 * 0.0625]
    for ch_axis, n in [(None, 1), (0, 6), (1, 40), (2, 9)]:
        s = np.full(n, 0.0625, np.float32) if ch_axis is None else rng.uniform(
            0.01, 0.1, n).astype(np.float32)
        z = rng.integers(-5, 5, n).astype(np.float32)
        a = O.quantize(x, s, z, *QINT8, ch_axis=ch_axis)
        b = O.quantize(x, s, z, *QINT8, ch_axis=ch_axis, faithful=True)
        assert np.array_equal(a, b)
        assert np.array_equal(O.dequantize(a, s, z, ch_axis=ch_axis),
                              O.dequantize(a, s, z, ch_axis=ch_axis, faithful=True))
        fa = O.fake_quantize(x, s, z, *QINT8, ch_axis=ch_axis)
        fb = O.fake_quantize(x, s, z, *QINT8, ch_axis=ch_axis, faithful=True)
        assert np.array_equal(fa.view(np.uint32), fb.view(np.uint32))


def test_code_offset_recentres():
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1000).astype(np.float32)
    q16 = O.quantize(x, 0.02, 131.0, *QUINT8, q_dtype=O.I16)
    q8 = O.quantize(x, 0.02, 131.0, *QUINT8, q_dtype=O.I8, code_offset=-128)
    assert np.array_equal(q8.astype(np.int16) + 128, q16)
    assert np.array_equal(O.dequantize(q8, 0.02, 131.0, code_offset=-128),
                          O.dequantize(q16, 0.02, 131.0))


# ------------------------------------------------------------------ torch cross-check
def test_codes_match_torch_quantize_per_tensor():
    # lucid/test/parity/quantization/test_functional_parity.py:20-28
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(0).standard_normal((3, 16)).astype(np.float32)
    ref = torch.quantize_per_tensor(torch.from_numpy(x), 0.05, 0, torch.qint8).int_repr().numpy()
    assert np.array_equal(O.quantize(x, 0.05, 0.0, *QINT8), ref)


@pytest.mark.parametrize("seed,shape,s,z,grid", [
    (2, (3, 16), 0.037, 0, QINT8),       # test_functional_parity.py:44-57
    (3, (5, 7), 0.02, 128, QUINT8),      # :59-70
])
def test_fake_quantize_matches_torch(seed, shape, s, z, grid):
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(seed).standard_normal(shape).astype(np.float32)
    ref = torch.fake_quantize_per_tensor_affine(torch.from_numpy(x), s, z, grid[0], grid[1])
    assert np.allclose(O.fake_quantize(x, s, float(z), *grid), ref.numpy(), atol=1e-4)


def test_fake_quantize_per_channel_matches_torch():
    # test_functional_parity.py:72-87
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(4).standard_normal((4, 8)).astype(np.float32)
    s = np.array([0.02, 0.03, 0.05, 0.017], np.float32)
    ref = torch.fake_quantize_per_channel_affine(
        torch.from_numpy(x), torch.from_numpy(s), torch.zeros(4, dtype=torch.int32), 0, -128, 127)
    got = O.fake_quantize(x, s, np.zeros(4, np.float32), *QINT8, ch_axis=0)
    assert np.allclose(got, ref.numpy(), atol=1e-4)


# ------------------------------------------------------------------ calculate_qparams
def test_qparams_affine_includes_zero():
    # test_functional.py:99-103
    s, z = O.calc_qparams(-1.0, 3.0, False, *QUINT8, signed=False)
    assert s[0] == pytest.approx(4.0 / 255.0, rel=1e-5)
    assert 0.0 <= z[0] <= 255.0
    # closed form in float32
    s32 = np.float32(4.0) / np.float32(255.0)
    assert s[0] == s32
    assert z[0] == np.float32(0) - np.rint(np.float32(-1.0) / s32)


def test_qparams_docstring_example():
    # lucid/quantization/_qparams.py:171-173
    s, z = O.calc_qparams(-2.0, 6.0, False, *QUINT8, signed=False)
    assert (round(float(s[0]), 4), float(z[0])) == (0.0314, 64.0)


def test_qparams_symmetric():
    # test_functional.py:105-108 ; divisor (qmax - qmin)/2 = 127.5
    s, z = O.calc_qparams(-2.5, 2.0, True, *QINT8, signed=True)
    assert z[0] == 0.0 and s[0] == np.float32(2.5) / np.float32(127.5)
    s, z = O.calc_qparams(-2.5, 2.0, True, *QUINT8, signed=False)
    assert z[0] == 128.0  # (255 + 0 + 1) // 2


def test_qparams_degenerate_range():
    # test_functional.py:110-113
    s, _ = O.calc_qparams(0.0, 0.0, False, *QINT8, signed=True)
    assert s[0] == np.float32(1e-8) and s[0] > 0


def test_qparams_positive_only_range_extends_to_zero():
    s, z = O.calc_qparams(2.0, 6.0, False, *QUINT8, signed=False)
    assert s[0] == np.float32(6.0) / np.float32(255.0) and z[0] == 0.0


def test_qparams_per_channel_vector():
    # lucid/test/unit/quantization/test_observer.py:43-50
    w = np.array([[1.0, 2.0, 3.0], [-4.0, 0.5, 0.1]], np.float32)
    mn, mx = O.minmax(w, ch_axis=0)
    assert mn.tolist() == [1.0, -4.0] and mx.tolist() == [3.0, 0.5]
    s, z = O.calc_qparams(mn, mx, True, *QINT8, signed=True)
    assert s.shape == (2,) and z.tolist() == [0.0, 0.0]
    assert np.array_equal(s, np.array([3.0, 4.0], np.float32) / np.float32(127.5))


def test_qparams_match_torch_observer():
    # lucid/test/parity/quantization/test_observer_parity.py:24-41 (scale 1e-6, zp +-1)
    torch = pytest.importorskip("torch")
    from torch.ao.quantization.observer import MinMaxObserver
    rng = np.random.default_rng(0)
    obs = MinMaxObserver(dtype=torch.quint8, qscheme=torch.per_tensor_affine)
    lo, hi = np.float32(np.inf), np.float32(-np.inf)
    for _ in range(3):
        b = rng.standard_normal((4, 8)).astype(np.float32)
        obs(torch.from_numpy(b))
        mn, mx = O.minmax(b)
        lo, hi = min(lo, mn[0]), max(hi, mx[0])
    ts, tz = obs.calculate_qparams()
    s, z = O.calc_qparams(lo, hi, False, *QUINT8, signed=False)
    assert abs(float(ts) - float(s[0])) < 1e-6 and abs(int(tz) - int(z[0])) <= 1


# ------------------------------------------------------------------ min / max
def test_minmax_running_known_answer():
    # test_observer.py:12-17
    a = np.array([[-1.0, 2.0], [0.5, 3.0]], np.float32)
    b = np.array([[-2.0, 1.0]], np.float32)
    (mn1,), (mx1,) = O.minmax(a)
    (mn2,), (mx2,) = O.minmax(b)
    assert min(mn1, mn2) == -2.0 and max(mx1, mx2) == 3.0


def test_minmax_matches_numpy_all_axes():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((5, 6, 7)).astype(np.float32)
    mn, mx = O.minmax(x)
    assert mn[0] == x.min() and mx[0] == x.max()
    for ax in range(3):
        mn, mx = O.minmax(x, ch_axis=ax)
        other = tuple(i for i in range(3) if i != ax)
        assert np.array_equal(mn, x.min(axis=other)) and np.array_equal(mx, x.max(axis=other))


def test_minmax_propagates_nan():
    # lucid/_C/backend/cpu/Reduce.cpp:87-125
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    x[1, 2] = np.nan
    mn, mx = O.minmax(x)
    assert np.isnan(mn[0]) and np.isnan(mx[0])
    mn, mx = O.minmax(x, ch_axis=0)
    assert np.isnan(mn[1]) and np.isnan(mx[1]) and mn[0] == 0.0 and mx[2] == 11.0


def test_minmax_empty_is_identity():
    mn, mx = O.minmax(np.zeros((0,), np.float32))
    assert mn[0] == np.inf and mx[0] == -np.inf


# ------------------------------------------------------------------ float16
def test_f32_to_f16_matches_numpy_on_bit_patterns():
    rng = np.random.default_rng(11)
    bits = rng.integers(0, 2 ** 32, 400000, dtype=np.uint64).astype(np.uint32)
    # concentrate on the f16 range, its subnormals and its overflow edge
    special = np.array([0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x477fe000, 0x477ff000,
                        0x477fefff, 0x33800000, 0x33000000, 0x33000001, 0x387fc000, 0x38800000,
                        0x3f801000, 0x3f803000, 0x3f802fff, 0x3f801001], np.uint32)
    mid = (rng.uniform(-70000, 70000, 200000)).astype(np.float32).view(np.uint32)
    tiny = (rng.uniform(-1e-4, 1e-4, 200000)).astype(np.float32).view(np.uint32)
    x = np.concatenate([bits, special, mid, tiny]).view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        expect = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.f32_to_f16_bits(x), expect)


def test_f16_to_f32_all_patterns():
    h = np.arange(65536, dtype=np.uint16)
    expect = h.view(np.float16).astype(np.float32)
    got = np.array([O.lib().orc_f16_to_f32(int(v)) for v in h], np.float32)
    ok = np.isnan(expect) | (got.view(np.uint32) == expect.view(np.uint32))
    assert ok.all()
