"""GPU parity of the engine primitives (one library call per IBackend call), of the
quantization composites written in them, and of the eval-mode BatchNorm forward.

The primitives are IEEE float32 operations, so numpy's float32 arithmetic is their
oracle; the composites are checked against the oracle's ``*_faithful`` passes (the
reference's pass structure) and against the fused kernels, all bit for bit."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.quantization as Q
import oracle as O

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def same(got, exp):
    """Bit equality, except that any NaN equals any NaN (the sign and payload of a generated
    NaN differ between x86 and the GPU)."""
    nan = np.isnan(exp)
    return np.array_equal(np.isnan(got), nan) and np.array_equal(bits(got)[~nan], bits(exp)[~nan])


def _operands(rng, n):
    a = (rng.standard_normal(n) * 10).astype(np.float32)
    b = (rng.standard_normal(n) * 3).astype(np.float32)
    special = np.float32([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-42, -1e-42, 3.4e38, 0.5, 1.5, 2.5, -0.5, -1.5])
    k = special.size
    a[:k], b[:k] = special, special[::-1]
    a[k:2 * k], b[k:2 * k] = special, np.float32(2.0)
    return a, b


@pytest.mark.parametrize("n", [1, 7, 1024, 100003])
def test_binary_primitives_are_ieee(n):
    rng = np.random.default_rng(n)
    a, b = _operands(rng, max(n, 32))
    a, b = a[:n], b[:n]
    A, B = hip(a), hip(b)
    with np.errstate(all="ignore"):
        assert same((A + B).numpy(), a + b)
        assert same((A - B).numpy(), a - b)
        assert same((A * B).numpy(), a * b)
        assert same((A / B).numpy(), a / b)
    # maximum / minimum: a NaN in either operand gives NaN (numpy's maximum has the same rule)
    with np.errstate(all="ignore"):
        mx, mn = L.maximum(A, B).numpy(), L.minimum(A, B).numpy()
        emx, emn = np.maximum(a, b), np.minimum(a, b)
    nan = np.isnan(a) | np.isnan(b)
    assert np.array_equal(np.isnan(mx), nan) and np.array_equal(np.isnan(mn), nan)
    # +0 / -0 ties may pick either zero: compare values there, bits elsewhere
    assert np.array_equal(mx[~nan], emx[~nan]) and np.array_equal(mn[~nan], emn[~nan])


def test_round_clip_astype():
    rng = np.random.default_rng(3)
    x = np.concatenate([(rng.standard_normal(5000) * 200).astype(np.float32),
                        np.arange(-10, 10, dtype=np.float32) + 0.5,          # every tie
                        np.float32([np.nan, np.inf, -np.inf, 8388607.5, -0.4, 1e-40])])
    X = hip(x)
    assert same(L.round(X).numpy(), np.rint(x))
    c = L.clip(X, -128, 127).numpy()
    e = x.copy()
    e[x < np.float32(-128)] = -128
    e[x > np.float32(127)] = 127                                             # NaN falls through both tests
    assert same(c, e)
    # astype: float -> int8 / int16 / int32 truncates toward zero inside the range
    y = np.clip(np.rint(x[np.isfinite(x)]), -128, 127).astype(np.float32)
    Y = hip(y)
    for dt, npdt in ((L.int8, np.int8), (L.int16, np.int16), (L.int32, np.int32)):
        assert np.array_equal(Y.to(dt).numpy(), y.astype(npdt))
    frac = hip(np.float32([1.9, -1.9, 0.99, -0.99, 126.5]))
    assert np.array_equal(frac.to(L.int8).numpy(), np.int8([1, -1, 0, 0, 126]))
    # integer -> float32 and float32 <-> float16
    q = rng.integers(-128, 128, 3000).astype(np.int8)
    assert np.array_equal(hip(q).to(L.float32).numpy(), q.astype(np.float32))
    q16 = rng.integers(-32768, 32768, 3000).astype(np.int16)
    assert np.array_equal(hip(q16).to(L.float32).numpy(), q16.astype(np.float32))
    f = (rng.standard_normal(3000) * 100).astype(np.float32)
    h = hip(f).to(L.float16)
    assert np.array_equal(h.numpy().view(np.uint16), f.astype(np.float16).view(np.uint16))
    assert np.array_equal(h.to(L.float32).numpy(), f.astype(np.float16).astype(np.float32))
    # NaN and out-of-range map to 0 and the int32 limits (undefined in C; documented here)
    odd = hip(np.float32([np.nan, 3e9, -3e9]))
    assert np.array_equal(odd.to(L.int32).numpy(), np.int32([0, 2147483647, -2147483648]))


@pytest.mark.parametrize("shape,ch_axis", [((64, 256), None), ((33, 7, 5), 0), ((6, 33, 9), 1), ((4, 5, 16), 2),
                                           ((2, 3, 4, 5), 1)])
@pytest.mark.parametrize("qdtype", [Q.qint8, Q.quint8])
def test_the_composite_as_written_equals_the_faithful_oracle_and_the_fused_kernel(shape, ch_axis, qdtype):
    """clip(round(x / s) + z, qmin, qmax).to(storage) and (q.to(float32) - z) * s
    (lucid/quantization/_functional.py:180,281), operator by operator on device tensors."""
    rng = np.random.default_rng(sum(shape))
    x = (rng.standard_normal(shape) * 2).astype(np.float32)
    Cn = 1 if ch_axis is None else shape[ch_axis]
    s = rng.uniform(0.005, 0.05, Cn).astype(np.float32)
    z = rng.integers(qdtype.quant_min, qdtype.quant_max + 1, Cn).astype(np.float32)
    x.reshape(-1)[:40] = (np.arange(40, dtype=np.float32) - 20 + 0.5) * s[0]      # ties of channel 0
    X = hip(x)
    if ch_axis is None:
        S, Z = hip(s.reshape(())), hip(z.reshape(()))
    else:
        view = [1] * len(shape)
        view[ch_axis] = Cn
        S, Z = hip(s).reshape(view), hip(z).reshape(view)
    storage = L.int8 if qdtype.storage == "int8" else L.int16
    codes = L.clip(L.round(X / S) + Z, qdtype.quant_min, qdtype.quant_max).to(storage)
    oq = O.quantize(x, s, z, qdtype.quant_min, qdtype.quant_max, ch_axis=ch_axis,
                    q_dtype=O.I8 if qdtype.storage == "int8" else O.I16, faithful=True)
    assert codes.dtype is storage and np.array_equal(codes.numpy(), oq)
    sq, zq = (hip(s), hip(z)) if ch_axis is not None else (hip(s.reshape(())), hip(z.reshape(())))
    assert np.array_equal(Q.quantize(X, sq, zq, qdtype, ch_axis=ch_axis).numpy(), oq)
    assert np.array_equal(bits(Q.fake_quantize(X, sq, zq, qdtype.quant_min, qdtype.quant_max, ch_axis=ch_axis).numpy()),
                          bits(O.fake_quantize(x, s, z, qdtype.quant_min, qdtype.quant_max, ch_axis=ch_axis,
                                               faithful=True)))
    # dequantize composite
    deq = (codes.to(L.float32) - Z) * S
    assert np.array_equal(bits(deq.numpy()), bits(O.dequantize(oq, s, z, ch_axis=ch_axis, faithful=True)))
    # fake-quantize composite (_functional.py:311-313)
    q_pre = L.round(X / S) + Z
    dq = (L.clip(q_pre, qdtype.quant_min, qdtype.quant_max) - Z) * S
    ofq = O.fake_quantize(x, s, z, qdtype.quant_min, qdtype.quant_max, ch_axis=ch_axis, faithful=True)
    assert np.array_equal(bits(dq.numpy()), bits(ofq))


REDUCE_CASES = [((1000,), None), ((64, 256), None), ((64, 256), 1), ((64, 256), 0), ((8, 5000), 1),
                ((6, 33, 9), 1), ((6, 33, 9), (0, 2)), ((6, 33, 9), 2), ((6, 33, 9), 0), ((2, 3, 4, 5), (2, 3)),
                ((2, 3, 4, 5), (0, 1)), ((2, 1, 4, 5), (0, 2)), ((7,), 0)]


@pytest.mark.parametrize("shape,dim", REDUCE_CASES)
def test_reduce_min_max_over_axes(shape, dim):
    rng = np.random.default_rng(len(shape) * 100 + sum(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    X = hip(x)
    axis = dim if dim is None or isinstance(dim, int) else tuple(dim)
    assert np.array_equal(X.min(dim).numpy(), x.min(axis=axis))
    assert np.array_equal(X.max(dim).numpy(), x.max(axis=axis))
    assert X.max(dim, keepdim=True).shape == x.max(axis=axis, keepdims=True).shape
    # a NaN anywhere in a reduced run makes that output NaN (Reduce.cpp:87-125)
    x.reshape(-1)[x.size // 2] = np.nan
    got = hip(x).min(dim).numpy()
    assert np.array_equal(np.isnan(got), np.isnan(x.min(axis=axis)))
    keep = ~np.isnan(got)
    assert np.array_equal(got[keep], np.asarray(x.min(axis=axis))[keep])


def test_reduce_rejects_what_it_cannot_merge():
    X = hip(np.zeros((2, 3, 4, 5), np.float32))
    with pytest.raises(NotImplementedError):
        X.min((1, 3))
    with pytest.raises(ValueError):
        X.min(7)


def test_observer_composite_min_max_then_qparams():
    """MinMaxObserver's x.min() / x.max() (observer.py:363-375) through the reduce primitive
    feed calculate_qparams exactly as the fused lq_minmax does."""
    rng = np.random.default_rng(5)
    x = rng.standard_normal((128, 300)).astype(np.float32)
    X = hip(x)
    mn, mx = X.min(), X.max()
    omn, omx = O.minmax(x)
    assert mn.shape == () and np.array_equal(mn.numpy(), omn.reshape(())) and np.array_equal(mx.numpy(), omx.reshape(()))
    pmn, pmx = X.min(1), X.max(1)                      # PerChannel, ch_axis 0 (observer.py:634-653)
    omn, omx = O.minmax(x, ch_axis=0)
    assert np.array_equal(pmn.numpy(), omn) and np.array_equal(pmx.numpy(), omx)


@pytest.mark.parametrize("shape", [(5, 7), (3, 6, 50), (2, 16, 24, 24), (2, 5, 3, 9, 11), (4, 8, 4096), (1, 3, 5000)])
@pytest.mark.parametrize("affine", [True, False])
def test_batchnorm_eval_forward(shape, affine):
    rng = np.random.default_rng(sum(shape))
    Cn = shape[1]
    cls = {2: nn.BatchNorm1d, 3: nn.BatchNorm1d, 4: nn.BatchNorm2d, 5: nn.BatchNorm3d}[len(shape)]
    bn = cls(Cn, eps=1e-3, affine=affine).eval()
    m = rng.standard_normal(Cn).astype(np.float32)
    v = rng.uniform(0.05, 4.0, Cn).astype(np.float32)
    bn.register_buffer("running_mean", L.tensor(m))
    bn.register_buffer("running_var", L.tensor(v))
    g = b = None
    if affine:
        g, b = rng.uniform(0.5, 1.5, Cn).astype(np.float32), rng.standard_normal(Cn).astype(np.float32)
        bn.register_buffer("weight", L.tensor(g))
        bn.register_buffer("bias", L.tensor(b))
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    y = bn(hip(x)).numpy()
    assert np.array_equal(bits(y), bits(O.batchnorm_eval(x, m, v, g, b, 1e-3)))
    with pytest.raises(L.ShapeMismatch):
        bn(hip(np.zeros((2, Cn + 1) + shape[2:], np.float32)))
    bn.train()
    with pytest.raises(NotImplementedError, match="training"):
        bn(hip(x))


def _randomize_bn(bn, rng):
    n = bn.num_features
    bn.register_buffer("weight", L.tensor(rng.uniform(0.5, 1.5, n).astype(np.float32)))
    bn.register_buffer("bias", L.tensor(rng.standard_normal(n).astype(np.float32)))
    bn.register_buffer("running_mean", L.tensor(rng.standard_normal(n).astype(np.float32)))
    bn.register_buffer("running_var", L.tensor(rng.uniform(0.2, 2.0, n).astype(np.float32)))


@pytest.mark.parametrize("rank", [1, 2])
def test_conv_bn_fold_matches_the_unfused_model_on_the_device(rank):
    """lucid/test/unit/quantization/test_static_ptq.py:90-99: fuse_modules([["conv", "bn"]]) on an
    eval-mode net gives the un-fused net's output (atol 1e-4), both run on the device."""
    rng = np.random.default_rng(rank)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nn.Conv2d(3, 8, 3, padding=1) if rank == 2 else nn.Conv1d(3, 8, 3, padding=1)
            self.bn = nn.BatchNorm2d(8) if rank == 2 else nn.BatchNorm1d(8)
            self.relu = nn.ReLU()

        def forward(self, x):
            return self.relu(self.bn(self.conv(x)))

    net = Net().eval()
    _randomize_bn(net.bn, rng)
    x = hip(rng.standard_normal((2, 3, 8, 8) if rank == 2 else (2, 3, 40)).astype(np.float32))
    y_ref = net(x).numpy()
    # the un-fused forward is conv, then the oracle's BatchNorm, then ReLU
    conv_out = net.conv(x).numpy()
    exp = np.maximum(O.batchnorm_eval(conv_out, net.bn.running_mean.numpy(), net.bn.running_var.numpy(),
                                      net.bn.weight.numpy(), net.bn.bias.numpy(), net.bn.eps), 0)
    assert np.array_equal(bits(y_ref), bits(exp))
    fused = Q.fuse_modules(net, [["conv", "bn"]])
    assert isinstance(fused.bn, nn.Identity)
    assert np.allclose(fused(x).numpy(), y_ref, atol=1e-4)
    assert np.abs(y_ref).max() > 0.5                         # not a comparison of zeros
    fused = Q.fuse_modules(net, [["conv", "bn", "relu"]])
    assert np.allclose(fused(x).numpy(), y_ref, atol=1e-4)


def test_unfused_conv_bn_model_calibrates_and_converts_after_fusion():
    """test_static_ptq.py:113-128: fuse, wrap, prepare, calibrate on the device, convert; the int8
    model tracks the un-fused float model run on the device."""
    import lucid_amd.nn.quantized as nnq
    rng = np.random.default_rng(3)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.conv = nn.Conv2d(3, 8, 3, padding=1)
            self.bn = nn.BatchNorm2d(8)
            self.relu = nn.ReLU()

        def forward(self, x):
            return self.relu(self.bn(self.conv(x)))

    net = Net().eval()
    _randomize_bn(net.bn, rng)
    fused = Q.fuse_modules(net, [["conv", "bn"]])
    prepared = Q.prepare(nnq.QuantWrapper(fused))
    for _ in range(8):
        prepared(hip(rng.standard_normal((4, 3, 8, 8)).astype(np.float32)))
    qm = Q.convert(prepared)
    assert isinstance(qm.module.conv, nnq.Conv2d) and qm.module.conv.weight_int8.dtype is L.int8
    xe = hip(rng.standard_normal((8, 3, 8, 8)).astype(np.float32))
    yf, yq = net(xe).numpy(), qm(xe).numpy()
    assert np.abs(yf - yq).mean() / (np.abs(yf).mean() + 1e-9) < 0.05
