"""GPU parity: quantize / dequantize / fake_quantize / minmax /
calculate_qparams on the hip device against the CPU oracle, bit for bit.

The first block restates the reference's own unit tests
(lucid/test/unit/quantization/test_functional.py, test_observer.py) against
this backend; the rest compares with the oracle on seeded and adversarial
inputs and checks size-independent properties at the benchmark's full size.
"""

import zlib

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.quantization as Q
import oracle as O

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.asarray(a), device="hip")


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def same_f32(a, b):
    """Bit-equal float32 arrays; NaNs match each other whatever their sign or
    payload (Lucid's own NaN bits come from Accelerate and are not pinned)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and bool(((bits(a) == bits(b)) | (np.isnan(a) & np.isnan(b))).all())


# ------------------------------------------------------------------ reference unit tests
class TestQuantizeDequantize:
    def test_round_trip_on_grid(self):
        x = hip([-1.0, -0.3, 0.0, 0.7, 2.0])
        q = Q.quantize(x, 0.05, 0.0, Q.qint8)
        assert q.dtype is L.int8
        dq = Q.dequantize(q, 0.05, 0.0)
        assert np.allclose(dq.numpy(), x.numpy(), atol=1e-6)

    def test_saturation(self):
        q = Q.quantize(hip([-1000.0, 1000.0]), 0.1, 0.0, Q.qint8)
        assert q.numpy().tolist() == [-128, 127]

    def test_affine_zero_point(self):
        q = Q.quantize(hip([0.0]), 0.02, 128.0, Q.quint8)
        assert q.dtype is L.int16 and q.item() == 128

    def test_docstring_example(self):
        assert Q.quantize(hip([100.0]), 0.05, 0.0, Q.qint8).item() == 127


class TestFakeQuantize:
    def test_equals_dequant_of_quant(self):
        x = hip([-1.0, -0.31, 0.0, 0.72, 2.0])
        fq = Q.fake_quantize(x, 0.05, 0.0, Q.qint8.quant_min, Q.qint8.quant_max)
        dq = Q.dequantize(Q.quantize(x, 0.05, 0.0, Q.qint8), 0.05, 0.0)
        assert np.array_equal(fq.numpy(), dq.numpy())


class TestPerChannel:
    def test_round_trip(self):
        w = hip([[1.0, 2.0, 3.0], [-4.0, 0.5, 0.1]])
        scale, zp = hip([0.03, 0.05]), hip([0.0, 0.0])
        q = Q.quantize(w, scale, zp, Q.qint8, ch_axis=0)
        dq = Q.dequantize(q, scale, zp, ch_axis=0)
        err = np.abs(dq.numpy() - w.numpy())
        assert (err <= np.array([[0.03 / 2], [0.05 / 2]]) + 1e-6).all()


class TestCalculateQParams:
    def test_affine_includes_zero(self):
        scale, zp = Q.calculate_qparams(-1.0, 3.0, Q.per_tensor_affine, Q.quint8)
        assert scale.item() == pytest.approx(4.0 / 255.0, rel=1e-5)
        assert 0.0 <= zp.item() <= 255.0

    def test_docstring_example(self):
        scale, zp = Q.calculate_qparams(-2.0, 6.0, Q.per_tensor_affine, Q.quint8)
        assert (round(scale.item(), 4), zp.item()) == (0.0314, 64.0)

    def test_symmetric_zero_point_pinned(self):
        scale, zp = Q.calculate_qparams(-2.5, 2.0, Q.per_tensor_symmetric, Q.qint8)
        assert zp.item() == 0.0 and scale.item() > 0.0

    def test_degenerate_range_floored(self):
        scale, _ = Q.calculate_qparams(0.0, 0.0, Q.per_tensor_affine, Q.qint8)
        assert scale.item() > 0.0

    @pytest.mark.parametrize("sym,qd", [(False, Q.quint8), (True, Q.qint8), (True, Q.quint8),
                                        (False, Q.qint8)])
    def test_vector_matches_oracle(self, sym, qd):
        rng = np.random.default_rng(0)
        mn = (rng.standard_normal(1000) * 3).astype(np.float32)
        mx = mn + np.abs(rng.standard_normal(1000)).astype(np.float32) * 4
        mn[:5] = [0, 1, -np.inf, np.nan, -1e-30]
        mx[:5] = [0, 2, np.inf, 1, 1e-30]
        scheme = {(False): Q.per_channel_affine, (True): Q.per_channel_symmetric}[sym]
        s, z = Q.calculate_qparams(hip(mn), hip(mx), scheme, qd)
        es, ez = O.calc_qparams(mn, mx, sym, qd.quant_min, qd.quant_max, qd.signed)
        assert same_f32(s.numpy(), es)
        assert same_f32(z.numpy(), ez)


# ------------------------------------------------------------------ oracle parity
SHAPES = [
    ((3, 16), None), ((5, 7), None), ((2, 10), None), ((4, 8), 0),       # reference parity shapes
    ((64, 784), None), ((256, 784), 0), ((10, 256), 0),                  # MLP config
    ((7, 33, 5), 1), ((7, 33, 5), 2), ((7, 33, 5), 0), ((6, 5, 1024), 1),
    ((3, 4, 2048), 0), ((1, 8200), None), ((2, 3, 5000), 1), ((64, 3, 7, 7), 0),
    ((1,), None), ((0,), None), ((4, 0), 0),
    ((16, 4096), 0), ((33, 1028), 0), ((2, 70000), None),
]


def _params(rng, shape, ch_axis, unsigned):
    n = 1 if ch_axis is None else shape[ch_axis]
    s = rng.uniform(0.004, 0.09, n).astype(np.float32)
    z = rng.integers(0, 255, n).astype(np.float32) if unsigned else \
        rng.integers(-10, 10, n).astype(np.float32)
    return s, z


def _adversarial(rng, shape, s0):
    x = (rng.standard_normal(shape) * 2.5).astype(np.float32)
    f = x.reshape(-1)
    if f.size >= 64:
        f[::13] *= 40                                       # saturating values
        k = np.arange(0, min(f.size, 4000), 7)
        f[k] = ((k % 300 - 150) + 0.5).astype(np.float32) * s0   # near or on ties
        f[3:14] = [np.inf, -np.inf, 0.0, -0.0, 1e-42, -1e-42, 3.4e38, -3.4e38, 1e-30, s0 / 2,
                   -s0 / 2]
    return x


@pytest.mark.parametrize("shape,ch_axis", SHAPES)
@pytest.mark.parametrize("qd", [Q.qint8, Q.quint8])
def test_quantize_family_bit_exact(shape, ch_axis, qd):
    rng = np.random.default_rng(zlib.crc32(repr((shape, ch_axis, qd.name)).encode()))
    s, z = _params(rng, shape, ch_axis, not qd.signed)
    x = _adversarial(rng, shape, s[0])
    xs = hip(x)
    if ch_axis is None:
        st, zt = float(s[0]), float(z[0])         # Python scalars, as Lucid callers pass them
    else:
        st, zt = hip(s), hip(z)
    q = Q.quantize(xs, st, zt, qd, ch_axis=ch_axis)
    q_dtype = O.I8 if qd.storage == "int8" else O.I16
    eq = O.quantize(x, s, z, qd.quant_min, qd.quant_max, ch_axis=ch_axis, q_dtype=q_dtype)
    assert q.shape == x.shape and np.array_equal(q.numpy(), eq)
    dq = Q.dequantize(q, st, zt, ch_axis=ch_axis)
    assert np.array_equal(bits(dq.numpy()), bits(O.dequantize(eq, s, z, ch_axis=ch_axis)))
    fq = Q.fake_quantize(xs, st, zt, qd.quant_min, qd.quant_max, ch_axis=ch_axis)
    assert np.array_equal(bits(fq.numpy()),
                          bits(O.fake_quantize(x, s, z, qd.quant_min, qd.quant_max, ch_axis=ch_axis)))


def test_device_scalar_qparams_equal_python_scalars():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((8, 512)) * 3).astype(np.float32)
    a = Q.quantize(hip(x), 0.037, 3.0, Q.qint8).numpy()
    b = Q.quantize(hip(x), hip(np.float32(0.037)), hip(np.float32(3.0)), Q.qint8).numpy()
    assert np.array_equal(a, b) and np.array_equal(a, O.quantize(x, 0.037, 3.0, -128, 127))


@pytest.mark.parametrize("s", [0.5, 2.0 ** -7, 1.0])
def test_ties_round_half_even_on_device(s):
    n = np.arange(-400, 401)
    x = ((n + 0.5) * s).astype(np.float32)
    x = np.tile(x, 3)[:2400]
    got = Q.quantize(hip(x), s, 128.0, Q.quint8).numpy()
    half_even = np.where(n % 2 == 0, n, n + 1)
    assert np.array_equal(got, np.tile(np.clip(half_even + 128, 0, 255), 3)[:2400])


def test_division_is_correctly_rounded_on_device():
    rng = np.random.default_rng(123)
    for _ in range(4):
        s = np.float32(rng.uniform(0.01, 0.2))
        n = rng.integers(-127, 127, 1 << 16)
        x = ((n + 0.5) * np.float64(s)).astype(np.float32)
        got = Q.quantize(hip(x), float(s), 0.0, Q.qint8).numpy()
        assert np.array_equal(got, O.quantize(x, s, 0.0, -128, 127))


def test_recentred_int8_storage_through_the_abi():
    from lucid_amd import _C
    rng = np.random.default_rng(3)
    x = rng.standard_normal(4096 * 3).astype(np.float32)
    xs = hip(x)
    q = L.Tensor.empty(x.shape, L.int8, "hip")
    s, z = hip(np.float32(0.02)), hip(np.float32(131.0))
    _C.call("lq_quantize", xs.data_ptr, q.data_ptr, _C.I8, -128, 1, 1, x.size, s.data_ptr,
            z.data_ptr, 0, 0, 255, None)
    assert np.array_equal(q.numpy(), O.quantize(x, 0.02, 131.0, 0, 255, code_offset=-128))
    out = L.Tensor.empty(x.shape, L.float32, "hip")
    _C.call("lq_dequantize", q.data_ptr, _C.I8, -128, out.data_ptr, 1, 1, x.size, s.data_ptr,
            z.data_ptr, 0, None)
    assert np.array_equal(bits(out.numpy()),
                          bits(O.dequantize(q.numpy(), 0.02, 131.0, code_offset=-128)))


def test_abi_rejects_bad_arguments():
    from lucid_amd import _C
    x = hip(np.zeros(16, np.float32))
    q = L.Tensor.empty((16,), L.int8, "hip")
    s = hip(np.ones(2, np.float32))
    with pytest.raises(L.DtypeMismatch):
        _C.call("lq_quantize", x.data_ptr, q.data_ptr, _C.F32, 0, 1, 1, 16, s.data_ptr, s.data_ptr,
                0, -128, 127, None)
    with pytest.raises(ValueError):   # quint8 grid does not fit int8 storage without the offset
        _C.call("lq_quantize", x.data_ptr, q.data_ptr, _C.I8, 0, 1, 1, 16, s.data_ptr, s.data_ptr,
                0, 0, 255, None)
    with pytest.raises(L.ShapeMismatch):
        Q.quantize(x, s, s, Q.qint8)          # 2 scales, no ch_axis
    with pytest.raises(L.ShapeMismatch):
        Q.quantize(x.reshape(4, 4), s, s, Q.qint8, ch_axis=0)   # 2 scales, 4 channels


# ------------------------------------------------------------------ min / max
class TestObserverStatistics:
    def test_running_minmax_known_answer(self):
        # lucid/test/unit/quantization/test_observer.py:12-17
        mn1, mx1 = Q.minmax(hip([[-1.0, 2.0], [0.5, 3.0]]))
        mn2, mx2 = Q.minmax(hip([[-2.0, 1.0]]))
        assert min(mn1.item(), mn2.item()) == -2.0 and max(mx1.item(), mx2.item()) == 3.0

    def test_per_channel_known_answer(self):
        # test_observer.py:43-50
        mn, mx = Q.minmax(hip([[1.0, 2.0, 3.0], [-4.0, 0.5, 0.1]]), ch_axis=0)
        assert mn.numpy().tolist() == [1.0, -4.0] and mx.numpy().tolist() == [3.0, 0.5]
        s, z = Q.calculate_qparams(mn, mx, Q.per_channel_symmetric, Q.qint8)
        assert s.shape == (2,) and z.numpy().tolist() == [0.0, 0.0]


@pytest.mark.parametrize("shape,ch_axis", [
    ((64, 784), None), ((256, 784), 0), ((5, 6, 7), 0), ((5, 6, 7), 1), ((5, 6, 7), 2),
    ((3, 4, 2048), 1), ((2, 3, 70000), 1), ((1, 300000), None), ((4100, 3), 1), ((1000, 8, 2), 1),
    ((16, 4096), 0), ((33, 1030), 0), ((1,), None), ((0,), None), ((3, 64, 56, 56), 1),
    ((40000, 16), 1),
])
def test_minmax_matches_oracle(shape, ch_axis):
    rng = np.random.default_rng(len(shape) * 100 + (ch_axis or 0))
    x = rng.standard_normal(shape).astype(np.float32)
    mn, mx = Q.minmax(hip(x), ch_axis=ch_axis)
    emn, emx = O.minmax(x, ch_axis=ch_axis)
    assert np.array_equal(mn.numpy().reshape(-1), emn)
    assert np.array_equal(mx.numpy().reshape(-1), emx)


def test_minmax_propagates_nan():
    x = np.arange(3 * 5000, dtype=np.float32).reshape(3, 5000)
    x[1, 4321] = np.nan
    mn, mx = Q.minmax(hip(x))
    assert np.isnan(mn.item()) and np.isnan(mx.item())
    mn, mx = Q.minmax(hip(x), ch_axis=0)
    assert np.isnan(mn.numpy()[1]) and mn.numpy()[0] == 0.0 and mx.numpy()[2] == 14999.0
    mn, mx = Q.minmax(hip(x.T.copy()), ch_axis=1)
    assert np.isnan(mx.numpy()[1]) and mn.numpy()[0] == 0.0 and mx.numpy()[2] == 14999.0


# ------------------------------------------------------------------ full-size properties
def test_round_trip_properties_at_benchmark_size():
    """4096 x 4096 x 16 float32, per-channel symmetric along dim 0, then
    per-tensor affine - checked through properties that hold at any size, and
    against the oracle on sampled channels."""
    from lucid_amd import _C
    shape = (4096, 4096, 16)
    n = int(np.prod(shape))
    x = L.Tensor.empty(shape, L.float32, "hip")
    _C.call("lq_fill_normal", x.data_ptr, n, 2, 0.001, 20.0, None)

    mn, mx = Q.minmax(x, ch_axis=0)
    s, z = Q.calculate_qparams(mn, mx, Q.per_channel_symmetric, Q.qint8)
    q = Q.quantize(x, s, z, Q.qint8, ch_axis=0)
    dq = Q.dequantize(q, s, z, ch_axis=0)
    # idempotence: a dequantized tensor quantizes back to the same codes
    q2 = Q.quantize(dq, s, z, Q.qint8, ch_axis=0)
    sh, mnh, mxh = s.numpy(), mn.numpy(), mx.numpy()
    for c in (0, 1, 2047, 4095):
        sl = slice(c * 65536, (c + 1) * 65536)
        xc = _slice_to_host(x, sl, np.float32)
        qc = _slice_to_host(q, sl, np.int8)
        assert mnh[c] == xc.min() and mxh[c] == xc.max()
        assert sh[c] == max(abs(mnh[c]), abs(mxh[c])) / np.float32(127.5)
        assert np.array_equal(qc, O.quantize(xc, sh[c], 0.0, -128, 127))
        dc = _slice_to_host(dq, sl, np.float32)
        assert np.array_equal(bits(dc), bits(O.dequantize(qc, sh[c], 0.0)))
        assert np.abs(dc - xc).max() <= sh[c] / 2 * (1 + 1e-4)   # nothing saturates
        assert np.array_equal(_slice_to_host(q2, sl, np.int8), qc)
    del q2, dq

    gmn, gmx = Q.minmax(x)
    assert gmn.item() == mnh.min() and gmx.item() == mxh.max()   # min of per-channel mins
    ts, tz = Q.calculate_qparams(gmn, gmx, Q.per_tensor_affine, Q.quint8)
    qt = Q.quantize(x, ts, tz, Q.quint8)
    assert qt.dtype is L.int16
    sl = slice(123 * 65536, 124 * 65536)
    xc = _slice_to_host(x, sl, np.float32)
    assert np.array_equal(_slice_to_host(qt, sl, np.int16),
                          O.quantize(xc, ts.item(), tz.item(), 0, 255, q_dtype=O.I16))


def _slice_to_host(t, sl, np_dtype):
    from lucid_amd import _C
    out = np.empty(sl.stop - sl.start, np_dtype)
    _C.call("lq_d2h", out.ctypes.data, t.data_ptr + sl.start * out.itemsize, out.nbytes, None)
    return out


@pytest.mark.parametrize("rows,cols", [(1, 4), (7, 784), (64, 1024), (33, 4096), (5, 16384), (3, 4100), (2, 20000),
                                       (9, 1028), (6, 2048), (2048, 4096)])
@pytest.mark.parametrize("scheme", ["sym_i8", "affine_u8", "affine_i8"])
def test_quantize_rows_dynamic_equals_the_three_calls_and_the_oracle(rows, cols, scheme):
    """One pass per row (min / max -> qparams -> codes) against minmax + calculate_qparams +
    quantize on the device and against the oracle; rows with outliers, constant rows, a NaN row."""
    import oracle as O
    rng = np.random.default_rng(rows * 31 + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    x[rng.random((rows, cols)) < 0.001] *= 20
    if rows > 2:
        x[1] = 0.25          # a constant row
        x[2, cols // 2] = np.nan
    qscheme, qdtype = {"sym_i8": (Q.per_channel_symmetric, Q.qint8), "affine_u8": (Q.per_channel_affine, Q.quint8),
                       "affine_i8": (Q.per_channel_affine, Q.qint8)}[scheme]
    xt = L.tensor(x, device="hip")
    if qdtype is Q.quint8:   # int16 storage: the wrapper takes the three-call route
        q, s, z = Q.quantize_rows_dynamic(xt, qscheme, qdtype)
    else:
        q, s, z = Q.quantize_rows_dynamic(xt, qscheme, qdtype)
    mn, mx = Q.minmax(xt, ch_axis=0)
    s3, z3 = Q.calculate_qparams(mn, mx, qscheme, qdtype)
    q3 = Q.quantize(xt, s3, z3, qdtype, ch_axis=0)
    assert np.array_equal(s.numpy().view(np.uint32), s3.numpy().view(np.uint32))
    assert np.array_equal(z.numpy().view(np.uint32), z3.numpy().view(np.uint32))
    assert np.array_equal(q.numpy(), q3.numpy())
    omn, omx = O.minmax(x, ch_axis=0)
    os_, oz = O.calc_qparams(omn, omx, qscheme.is_symmetric, qdtype.quant_min, qdtype.quant_max, qdtype.signed)
    ok = ~np.isnan(os_)
    assert np.array_equal(s.numpy()[ok].view(np.uint32), os_[ok].view(np.uint32))
    oq = O.quantize(x, os_, oz, qdtype.quant_min, qdtype.quant_max, ch_axis=0,
                    q_dtype=O.I8 if qdtype.storage == "int8" else O.I16)
    assert np.array_equal(q.numpy()[ok], oq[ok])


@pytest.mark.parametrize("n", [0, 1, 3, 4, 1000, 64 * 784, 262144, 50177])
@pytest.mark.parametrize("qd", ["quint8", "qint8"])
def test_quantize_tensor_dynamic_equals_the_three_calls(n, qd):
    """Global min / max, qparams and codes of a small tensor in one launch: the bits of
    minmax + calculate_qparams + quantize (and so of the oracle, which those are tested against)."""
    from lucid_amd import _C
    rng = np.random.default_rng(n + len(qd))
    x = (rng.standard_normal(n) * 3 + 0.5).astype(np.float32)
    qdtype = getattr(Q, qd)
    off = -128 if qd == "quint8" else 0
    xt = L.tensor(x, device="hip")
    q = L.Tensor.empty((n,), L.int8, "hip")
    s, z = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
    mn1, mx1 = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
    _C.call("lq_quantize_tensor_dynamic_i8", xt.data_ptr if n else None, n, 0, qdtype.quant_min, qdtype.quant_max,
            int(qdtype.signed), 1e-8, off, s.data_ptr, z.data_ptr, mn1.data_ptr, mx1.data_ptr,
            q.data_ptr if n else None, None)
    mn, mx = Q.minmax(xt)
    s3, z3 = Q.calculate_qparams(mn, mx, Q.per_tensor_affine, qdtype)
    assert np.array_equal(bits(mn1.numpy()), bits(mn.numpy())) and np.array_equal(bits(mx1.numpy()), bits(mx.numpy()))
    assert np.array_equal(bits(s.numpy()), bits(s3.numpy())) and np.array_equal(bits(z.numpy()), bits(z3.numpy()))
    if n:
        q3 = L.Tensor.empty((n,), L.int8, "hip")
        _C.call("lq_quantize", xt.data_ptr, q3.data_ptr, _C.I8, off, 1, 1, n, s3.data_ptr, z3.data_ptr, 0,
                qdtype.quant_min, qdtype.quant_max, None)
        assert np.array_equal(q.numpy(), q3.numpy())
        exp = O.quantize(x, s3.numpy(), z3.numpy(), qdtype.quant_min, qdtype.quant_max, code_offset=off)
        assert np.array_equal(q.numpy(), exp)


def test_quantize_tensor_dynamic_refuses_large_tensors():
    from lucid_amd import _C
    x = L.Tensor.empty((262145,), L.float32, "hip")
    q = L.Tensor.empty((262145,), L.int8, "hip")
    s, z = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
    with pytest.raises(NotImplementedError):
        _C.call("lq_quantize_tensor_dynamic_i8", x.data_ptr, 262145, 0, 0, 255, 0, 1e-8, -128, s.data_ptr, z.data_ptr,
                None, None, q.data_ptr, None)
