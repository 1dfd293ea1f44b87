"""Group-wise weight-only int4 / int8 on the device against the restatement
(oracle/wq_group.py) and the reference's own tests for this path
(lucid/test/unit/quantization/test_real_gemm.py)."""

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn as nn
import lucid_amd.nn.quantized as nnq
import oracle.wq_group as W
from lucid_amd.quantization import _qgemm

pytestmark = pytest.mark.gpu


def hip(a):
    return L.tensor(a, device="hip")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("N,K", [(24, 256), (11008, 4096), (7, 128)])
def test_quantize_and_dequantize_bit_exact(bits, gs, N, K):
    rng = np.random.default_rng(bits + gs + N)
    w = rng.standard_normal((N, K)).astype(np.float32)
    packed, s, b = _qgemm.quantize(hip(w), gs, bits)
    ep, es, eb = W.quantize(w, gs, bits)
    assert packed.shape == ep.shape and packed.dtype is L.int32
    assert np.array_equal(packed.numpy(), ep)
    assert np.array_equal(s.numpy(), es) and np.array_equal(b.numpy(), eb)
    deq = _qgemm.dequantize(packed, s, b, gs, bits).numpy()
    assert np.array_equal(deq, W.dequantize(ep, es, eb, gs, bits))
    # half a step, plus the rounding of c * s + beta itself
    assert np.all(np.abs(deq - w) <= np.repeat(es, gs, axis=1) * 0.5 + 4e-7 * (1 + np.abs(w)))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,N,K,gs", [(1, 256, 512, 64), (3, 100, 256, 32), (4, 512, 4096, 128), (16, 64, 1024, 64),
                                      (8, 128, 128, 64), (40, 96, 256, 64), (2, 64, 8192, 64),
                                      # matrix-core path: ragged M and N, several row blocks, k steps not a
                                      # multiple of the four wavefronts, K too ragged for it (192 at 4 bits)
                                      (5, 33, 640, 32), (16, 11008, 4096, 64), (17, 70, 1152, 128),
                                      (64, 257, 2048, 64), (7, 48, 192, 32), (65, 64, 512, 64)])
def test_matmul_against_the_dequantize_path(bits, M, N, K, gs):
    rng = np.random.default_rng(bits * 7 + M + N + K)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    x = rng.standard_normal((M, K)).astype(np.float32)
    packed, s, b = _qgemm.quantize(hip(w), gs, bits)
    y = _qgemm.quantized_matmul(hip(x), packed, s, b, True, gs, bits).numpy()
    ref = W.matmul(x, packed.numpy(), s.numpy(), b.numpy(), gs, bits)
    assert y.shape == (M, N)
    assert np.abs(y - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())
    # test_real_gemm.py:80-94: fused kernel vs dequantize -> float matmul, atol 1e-3
    y_deq = x @ _qgemm.dequantize(packed, s, b, gs, bits).numpy().T
    assert np.allclose(y, y_deq, atol=1e-3)


@pytest.mark.parametrize("bits", [4, 8])
def test_small_batch_matmul_is_reproducible_and_exact_on_exact_inputs(bits):
    # the matrix-core path adds the partial sums of its k ranges in a fixed order: two calls
    # agree bit for bit; and with x, scales and biases that keep every product and sum exact in
    # float32 (small integers), the result equals the integer arithmetic exactly - x is split
    # into bfloat16 parts without loss and the codes enter unrounded
    rng = np.random.default_rng(bits)
    M, N, K, gs = 16, 300, 1024, 64
    packed = rng.integers(0, 2**32, (N, K * bits // 32), dtype=np.uint32).view(np.int32)
    s = rng.integers(1, 3, (N, K // gs)).astype(np.float32)
    b = rng.integers(-8, 9, (N, K // gs)).astype(np.float32)
    x = rng.integers(-7, 8, (M, K)).astype(np.float32)  # every partial sum stays below 2^24
    args = (hip(x), hip(packed), hip(s), hip(b), True, gs, bits)
    y1 = _qgemm.quantized_matmul(*args).numpy()
    y2 = _qgemm.quantized_matmul(*args).numpy()
    assert np.array_equal(y1, y2)
    w = W.dequantize(packed, s, b, gs, bits).astype(np.float64)
    assert np.array_equal(y1.astype(np.float64), x.astype(np.float64) @ w.T)


def test_decoding_takes_foreign_scales_and_biases_as_given():
    # a weight packed elsewhere under the same contract may carry negative scales
    rng = np.random.default_rng(1)
    packed = rng.integers(0, 2**32, (32, 16), dtype=np.uint32).view(np.int32)  # K = 128 at 4 bits
    s = rng.standard_normal((32, 2)).astype(np.float32) * 0.1
    b = rng.standard_normal((32, 2)).astype(np.float32)
    x = rng.standard_normal((2, 128)).astype(np.float32)
    y = _qgemm.quantized_matmul(hip(x), hip(packed), hip(s), hip(b), True, 64, 4).numpy()
    assert np.allclose(y, W.matmul(x, packed, s, b, 64, 4), atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("bits,bound", [(8, 0.02), (4, 0.15)])
def test_linear_module_accuracy_and_memory(bits, bound):
    # test_real_gemm.py:29-64
    lin = nn.Linear(256, 256)
    rng = np.random.default_rng(bits)
    x = rng.standard_normal((16, 256)).astype(np.float32)
    yf = x @ lin.weight.numpy().T + lin.bias.numpy()
    q = nnq.QuantizedLinearMLX.from_float(lin, bits=bits)
    yq = q(hip(x)).numpy()
    assert np.abs(yf - yq).max() / (np.abs(yf).max() + 1e-9) < bound
    packed_bytes = q.packed_weight.numpy().nbytes + q.scales.numpy().nbytes + q.biases.numpy().nbytes
    assert packed_bytes < 256 * 256 * 4 / 2
    qr = nnq.QuantizedLinearMLX.from_float(lin, bits=bits, relu=True)
    assert np.array_equal(qr(hip(x)).numpy(), np.maximum(yq, 0))


def test_state_dict_round_trip(tmp_path):
    # test_real_gemm.py:66-78: the int32-tagged packed weight survives save -> load
    for bits in (8, 4):
        lin = nn.Linear(128, 64)
        x = hip(np.random.default_rng(bits).standard_normal((8, 128)).astype(np.float32))
        q = nnq.QuantizedLinearMLX.from_float(lin, bits=bits)
        before = q(x).numpy()
        path = str(tmp_path / f"wq{bits}.lucid")
        L.save(q.state_dict(), path)
        q2 = nnq.QuantizedLinearMLX(128, 64, bits=bits)
        q2.load_state_dict(L.load(path))
        assert np.array_equal(before, q2(x).numpy())


def test_argument_validation():
    w = hip(np.zeros((4, 96), np.float32))
    with pytest.raises(_C_err()):
        _qgemm.quantize(w, 64, 8)  # 96 is not a multiple of 64
    with pytest.raises(ValueError):
        _qgemm.quantize(hip(np.zeros((4, 128), np.float32)), 64, 3)
    with pytest.raises(ValueError):
        _qgemm.quantize(hip(np.zeros((4, 128), np.float32)), 48, 8)


def _C_err():
    return L.ShapeMismatch


class TestConvertRoutesToGroupWise:
    """test_real_gemm.py:94-145, with the engine named explicitly: here ``"auto"``
    builds the int8 x int8 modules and ``"mlx_group"`` the weight-only ones."""

    @pytest.fixture(autouse=True)
    def _engine(self):
        L.backends.quantized.engine = "mlx_group"
        yield
        L.backends.quantized.engine = "auto"

    @staticmethod
    def _prepared(model, shapes_in, rng):
        import lucid_amd.quantization as Q
        prepared = Q.prepare(model, Q.get_default_qconfig())
        for mod in prepared.modules():
            if hasattr(mod, "activation_post_process"):
                mod.activation_post_process(hip(rng.standard_normal(shapes_in).astype(np.float32)))
        return prepared

    def test_static_convert_routes_linear(self):
        import lucid_amd.quantization as Q
        rng = np.random.default_rng(0)
        m = nn.Sequential(nn.Linear(128, 256), nn.ReLU(), nn.Linear(256, 64))
        x = rng.standard_normal((16, 128)).astype(np.float32)
        w0, b0, w2, b2 = (t.numpy() for t in (m[0].weight, m[0].bias, m[2].weight, m[2].bias))
        yf = np.maximum(x @ w0.T + b0, 0) @ w2.T + b2
        qm = Q.convert(self._prepared(m, (16, 64), rng))
        assert isinstance(qm[0], nnq.QuantizedLinearMLX) and isinstance(qm[2], nnq.QuantizedLinearMLX)
        assert qm[0].group_size == 64 and qm[0].bits == 8
        yq = qm(hip(x)).numpy()
        assert np.abs(yf - yq).max() / (np.abs(yf).max() + 1e-9) < 0.05

    def test_dynamic_convert_routes_linear(self):
        import lucid_amd.quantization as Q
        m = nn.Sequential(nn.Linear(96, 256), nn.ReLU(), nn.Linear(256, 64))
        qm = Q.quantize_dynamic(m)
        assert isinstance(qm[0], nnq.QuantizedLinearMLX) and qm[0].group_size == 32
        assert isinstance(qm[2], nnq.QuantizedLinearMLX) and qm[2].group_size == 64

    def test_indivisible_dim_keeps_the_int8_form(self):
        import lucid_amd.quantization as Q
        rng = np.random.default_rng(2)
        qm = Q.convert(self._prepared(nn.Sequential(nn.Linear(8, 16)), (4, 16), rng))
        assert isinstance(qm[0], nnq.Linear) and not isinstance(qm[0], nnq.QuantizedLinearMLX)
        import lucid_amd.nn.quantized.dynamic as nnqd
        assert isinstance(Q.quantize_dynamic(nn.Sequential(nn.Linear(8, 16)))[0], nnqd.Linear)

    def test_relu_fused_variant_routes(self):
        import lucid_amd.nn.intrinsic as nni
        import lucid_amd.quantization as Q
        rng = np.random.default_rng(3)
        m = nn.Sequential(nni.LinearReLU(nn.Linear(64, 128), nn.ReLU()))
        qm = Q.convert(self._prepared(m, (8, 128), rng))
        assert isinstance(qm[0], nnq.QuantizedLinearMLX) and qm[0].relu is True
        y = qm(hip(rng.standard_normal((8, 64)).astype(np.float32))).numpy()
        assert y.min() >= 0.0


def test_backends_toggle():
    # test_real_gemm.py:148-158
    q = L.backends.quantized
    assert q.engine == "auto" and not q.use_mlx()
    q.engine = "mlx_group"
    assert q.use_mlx()
    q.engine = "reference"
    assert not q.use_mlx()
    q.engine = "auto"
    with pytest.raises(ValueError):
        q.engine = "nonsense"
