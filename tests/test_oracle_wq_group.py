"""The group-wise weight-only restatement against the documented contract; CPU only."""

import numpy as np
import pytest

import oracle.wq_group as W


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("gs", [32, 64, 128])
def test_contract_properties(bits, gs):
    rng = np.random.default_rng(bits * 10 + gs)
    w = rng.standard_normal((24, 256)).astype(np.float32)
    packed, s, b = W.quantize(w, gs, bits)
    # shapes and density (_qgemm.py:122-125,141-147)
    assert packed.shape == (24, 256 * bits // 32) and packed.dtype == np.int32
    assert s.shape == b.shape == (24, 256 // gs)
    # bias is the group minimum, scale the step over the group's range
    g = w.reshape(24, 256 // gs, gs)
    assert np.array_equal(b, g.min(-1))
    assert np.allclose(s, (g.max(-1) - g.min(-1)) / ((1 << bits) - 1), rtol=1e-6)
    # codes use the whole grid and reconstruct within half a step (_qgemm.py:163-166)
    c = W.unpack(packed, bits)
    assert c.min() == 0 and c.max() == (1 << bits) - 1
    err = np.abs(W.dequantize(packed, s, b, gs, bits) - w)
    assert np.all(err <= np.repeat(s, gs, axis=1) * 0.5 + 4e-7 * (1 + np.abs(w)))  # + rounding of c * s + beta


def test_little_endian_packing_of_known_codes():
    # 8 four-bit codes 0..7 of one word: code j at bits [4j, 4j+4)
    w = np.arange(32, dtype=np.float32).reshape(1, 32) / 31 * 15  # 32 values on the 4-bit grid 0..15
    packed, s, b = W.quantize(w, 32, 4)
    assert s[0, 0] == pytest.approx(1.0, rel=1e-6) and b[0, 0] == 0.0
    codes = np.rint(w[0]).astype(np.uint32)
    for wd in range(4):
        word = sum(int(codes[wd * 8 + j]) << (4 * j) for j in range(8))
        assert packed.view(np.uint32)[0, wd] == word


def test_constant_group_decodes_exactly():
    w = np.full((2, 64), 0.37, np.float32)
    packed, s, b = W.quantize(w, 64, 8)
    assert np.array_equal(W.dequantize(packed, s, b, 64, 8), w)


@pytest.mark.parametrize("bits,bound", [(8, 0.02), (4, 0.15)])
def test_linear_accuracy_bounds_of_the_reference_tests(bits, bound):
    # test_real_gemm.py:29-52: nn.Linear(256, 256) default init, randn(16, 256)
    rng = np.random.default_rng(bits)
    k = 1 / np.sqrt(256)
    w = rng.uniform(-k, k, (256, 256)).astype(np.float32)
    x = rng.standard_normal((16, 256)).astype(np.float32)
    yf = x @ w.T
    yq = W.matmul(x, *W.quantize(w, 64, bits), 64, bits)
    assert np.abs(yf - yq).max() / np.abs(yf).max() < bound
