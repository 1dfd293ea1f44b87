"""GPU parity of the int8 GEMM + fused epilogue (``lq_qlinear_i8``) against
the CPU oracle: int32 accumulators and requantized codes bit for bit, float
outputs bit for bit as well (same float steps in the same order), on all three
kernels (tile / skinny / naive), ragged shapes and every output form."""

import numpy as np
import pytest

import lucid_amd as L
from lucid_amd import _ops
import oracle as O

pytestmark = pytest.mark.gpu

TILE, SKINNY, NAIVE = _ops.PATH_TILE, _ops.PATH_SKINNY, _ops.PATH_NAIVE


def hip(a):
    return L.tensor(np.ascontiguousarray(a), device="hip")


def codes(rng, shape, lo=-128, hi=127):
    return rng.integers(lo, hi + 1, shape).astype(np.int8)


ACC_CASES = [
    # M, N, K, path
    (256, 256, 128, TILE), (256, 256, 256, TILE), (512, 512, 4096, TILE), (300, 260, 144, TILE),
    (1, 16, 16, TILE), (129, 77, 784, TILE), (700, 1000, 576, TILE), (64, 256, 784, TILE),
    (1, 11008, 4096, SKINNY), (16, 11008, 4096, SKINNY), (16, 1024, 4096, SKINNY),
    (3, 50, 48, SKINNY), (17, 33, 784, SKINNY), (33, 100, 272, SKINNY), (64, 256, 784, SKINNY),
    (64, 10, 256, SKINNY), (5, 7, 16, SKINNY),
    # one activation row (dot-product kernel): ragged N, K tails, several 4 KiB chunks, few rows
    (1, 50, 48, SKINNY), (1, 4096, 11008, SKINNY), (1, 77, 4112, SKINNY), (1, 3, 16, SKINNY), (1, 1031, 1024, SKINNY),
    (1, 9000, 256, SKINNY), (1, 2, 65536, SKINNY),
    # 2..16 rows with K >= 1024 (one block per compute unit's share of the rows)
    (2, 11008, 4096, SKINNY), (7, 1000, 1040, SKINNY), (16, 4099, 2048, SKINNY), (9, 16400, 1024, SKINNY),
    (13, 33, 8192, SKINNY), (5, 12000, 1296, SKINNY), (3, 31, 6144, SKINNY), (16, 64, 2048, SKINNY), (4, 70, 1280, SKINNY), (2, 40, 16384, SKINNY), (8, 300, 8192, SKINNY),
    (5, 7, 3, NAIVE), (17, 33, 147, NAIVE), (64, 10, 250, NAIVE),
]


@pytest.mark.parametrize("M,N,K,path", ACC_CASES)
def test_accumulators_exact(M, N, K, path):
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    acc = _ops.qlinear_i8(hip(a), hip(w), out_mode=_ops.OUT_ACC_I32, path=path).numpy()
    assert np.array_equal(acc, O.igemm(a, w))


@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12])
@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 260, 144), (129, 77, 784), (513, 1000, 576),
                                   (2048, 512, 4096), (1, 16, 16), (700, 130, 64)])
def test_every_tile_shape_exact(cfg, M, N, K):
    rng = np.random.default_rng(cfg * 1000 + M + N + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    acc = _ops.qlinear_i8(hip(a), hip(w), out_mode=_ops.OUT_ACC_I32, path=TILE,
                          tile_config=cfg).numpy()
    assert np.array_equal(acc, O.igemm(a, w))
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    got = _ops.qlinear_i8(hip(a), hip(w), a_scale=hip(a_scale), w_scale=hip(w_scale),
                          bias=hip(bias), out_mode=_ops.OUT_F16, path=TILE, tile_config=cfg).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


@pytest.mark.parametrize("cfg", [1, 3, 4, 5, 6, 8, 9, 10, 11, 12])
@pytest.mark.parametrize("M,N,K", [(300, 260, 144), (513, 1000, 576), (2048, 1100, 4096),
                                   (256, 256, 128), (129, 77, 784), (1500, 3000, 1024)])
def test_stream_k_schedule_exact(cfg, M, N, K):
    """Forced stream-K work split: tiles shared between workers are finished by
    whoever arrives last; integer partial sums make the result exact.  Launched
    twice to show that the arrival counters are left reset."""
    rng = np.random.default_rng(cfg * 31 + M + N + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    ref = O.igemm(a, w)
    ad, wd = hip(a), hip(w)
    for _ in range(2):
        acc = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=TILE,
                              tile_config=cfg | 0x200).numpy()
        assert np.array_equal(acc, ref)
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    got = _ops.qlinear_i8(ad, wd, a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                          out_mode=_ops.OUT_F16, path=TILE, tile_config=cfg | 0x200).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


@pytest.mark.parametrize("cfg,M,N,K", [(4, 2048, 11008, 512), (5, 3000, 3000, 256), (6, 4096, 2500, 320),
                                       (3, 4096, 5000, 256), (4, 2100, 11000, 400), (1, 2048, 11008, 192)])
def test_hybrid_schedule_exact(cfg, M, N, K):
    """More tiles than fit on the chip at once: the leftover tiles of the last
    round are shared between all workers (partial sums met by the last arriver),
    the rest run one block per tile.  Launched twice: the arrival counters must
    be left reset."""
    rng = np.random.default_rng(cfg * 17 + M + N + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    ref = O.igemm(a, w)
    ad, wd = hip(a), hip(w)
    tc = cfg | 0x300
    for _ in range(2):
        acc = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=tc).numpy()
        assert np.array_equal(acc, ref)
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    got = _ops.qlinear_i8(ad, wd, a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                          out_mode=_ops.OUT_F16, path=TILE, tile_config=tc).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


@pytest.mark.parametrize("path,M", [(TILE, 300), (SKINNY, 16), (NAIVE, 9)])
def test_extreme_codes(path, M):
    K, N = 4096, 48
    a = np.full((M, K), -128, np.int8)
    w = np.full((N, K), -128, np.int8)
    acc = _ops.qlinear_i8(hip(a), hip(w), out_mode=_ops.OUT_ACC_I32, path=path).numpy()
    assert (acc == 128 * 128 * K).all()


def test_auto_path_matches_forced_paths():
    rng = np.random.default_rng(0)
    for M in (1, 16, 64, 65, 200):
        a, w = codes(rng, (M, 512)), codes(rng, (96, 512))
        ref = O.igemm(a, w)
        assert np.array_equal(_ops.qlinear_i8(hip(a), hip(w), out_mode=0).numpy(), ref)
    a, w = codes(rng, (20, 50)), codes(rng, (9, 50))     # K % 16 != 0 -> naive
    assert np.array_equal(_ops.qlinear_i8(hip(a), hip(w), out_mode=0).numpy(), O.igemm(a, w))


def _epilogue_case(rng, M, N, K, per_row, bias_kind):
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    a_scale = rng.uniform(0.005, 0.05, M if per_row else 1).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = None
    if bias_kind == "f32":
        bias = rng.standard_normal(N).astype(np.float32)
    elif bias_kind == "f16":
        bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    a_zp = 0 if per_row else int(rng.integers(-128, 127))
    return a, w, a_scale, w_scale, bias, a_zp


MODES = [_ops.OUT_F32, _ops.OUT_F16, _ops.OUT_REQUANT_I8, _ops.OUT_FAKEQUANT_F32]


@pytest.mark.parametrize("path,M,N,K", [(TILE, 300, 260, 144), (TILE, 64, 256, 784),
                                         (SKINNY, 16, 272, 4096), (SKINNY, 37, 50, 64),
                                         (SKINNY, 1, 1030, 4096), (SKINNY, 1, 45, 4112), (SKINNY, 11, 700, 2064),
                                         (NAIVE, 9, 21, 30)])
@pytest.mark.parametrize("per_row,bias_kind,relu", [(False, "f32", False), (False, "f32", True),
                                                    (True, "f16", False), (False, None, True),
                                                    (True, None, False)])
def test_epilogue_bit_exact(path, M, N, K, per_row, bias_kind, relu):
    rng = np.random.default_rng(M + 13 * N + K + int(per_row) + int(relu))
    a, w, a_scale, w_scale, bias, a_zp = _epilogue_case(rng, M, N, K, per_row, bias_kind)
    wsum = _ops.rowsum_i8(hip(w))
    assert np.array_equal(wsum.numpy(), O.rowsum_i8(w))
    y = O.qlinear(a, w, a_zp, a_scale, w_scale, bias=bias, relu=relu, out_mode=O.OUT_F32)
    S = np.float32(np.abs(y).max() / 200 + 1e-6)
    Z = np.float32(0.0 if relu else 128.0)
    for mode in MODES:
        got = _ops.qlinear_i8(hip(a), hip(w), a_zp=a_zp, a_scale=hip(a_scale),
                              w_scale=hip(w_scale), wsum=wsum,
                              bias=None if bias is None else hip(bias), relu=relu, out_mode=mode,
                              out_scale=hip(S), out_zp=hip(Z), out_qmin=0, out_qmax=255,
                              out_offset=-128, path=path).numpy()
        exp = O.qlinear(a, w, a_zp, a_scale, w_scale, bias=bias, relu=relu, out_mode=mode,
                        out_scale=S, out_zp=Z, out_qmin=0, out_qmax=255, out_offset=-128)
        if mode == _ops.OUT_F16:
            assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))
        elif mode == _ops.OUT_REQUANT_I8:
            assert np.array_equal(got, exp)
        else:
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))


def test_llm_shape_f16_output_matches_oracle_on_sampled_rows():
    """K=4096, N=11008 with per-token activation scales, per-row weight scales,
    fp16 bias, fp16 output - the benchmark's Linear, M = 2048 on the tile
    kernel and M = 1, 16 on the skinny kernel."""
    rng = np.random.default_rng(42)
    K, N = 4096, 11008
    wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    mn, mx = O.minmax(wf, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    wq = O.quantize(wf, ws, wz, -128, 127, ch_axis=0)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    w_dev, ws_dev, b_dev = hip(wq), hip(ws), hip(bias)
    for M in (1, 16, 2048):
        x = rng.standard_normal((M, K)).astype(np.float32)
        mn, mx = O.minmax(x, ch_axis=0)
        xs, xz = O.calc_qparams(mn, mx, True, -128, 127, True)
        xq = O.quantize(x, xs, xz, -128, 127, ch_axis=0)
        got = _ops.qlinear_i8(hip(xq), w_dev, a_scale=hip(xs), w_scale=ws_dev, bias=b_dev,
                              out_mode=_ops.OUT_F16).numpy()
        rows = np.unique(rng.integers(0, M, 24))
        exp = O.qlinear(xq[rows], wq, 0, xs[rows], ws, bias=bias, out_mode=O.OUT_F16)
        assert np.array_equal(got[rows].view(np.uint16), exp.view(np.uint16))
        # linearity of the exact accumulators at full size: acc(x, w) + acc(x', w) == acc(x + x', w)
        if M == 2048:
            xa = codes(rng, (M, K), -60, 60)
            xb = codes(rng, (M, K), -60, 60)
            acc = lambda t: _ops.qlinear_i8(hip(t), w_dev, out_mode=_ops.OUT_ACC_I32).numpy()
            assert np.array_equal(acc(xa) + acc(xb), acc((xa + xb).astype(np.int8)))


def test_argument_validation():
    a, w = hip(np.zeros((4, 32), np.int8)), hip(np.zeros((8, 32), np.int8))
    with pytest.raises(L.ShapeMismatch):
        _ops.qlinear_i8(a, hip(np.zeros((8, 16), np.int8)))
    with pytest.raises(ValueError):      # a_zp without the weight row sums
        _ops.qlinear_i8(a, w, a_zp=3, a_scale=hip(np.ones(1, np.float32)),
                        w_scale=hip(np.ones(8, np.float32)))
    with pytest.raises(L.DtypeMismatch):
        _ops.qlinear_i8(hip(np.zeros((4, 32), np.float32)), w)
    with pytest.raises(L.DeviceMismatch):
        _ops.qlinear_i8(L.tensor(np.zeros((4, 32), np.int8)), w)
    with pytest.raises(L.ShapeMismatch):  # skinny path forced on a tall problem
        _ops.qlinear_i8(hip(np.zeros((100, 32), np.int8)), w, out_mode=0, path=SKINNY)
    with pytest.raises(ValueError):       # MFMA path on K % 16 != 0
        _ops.qlinear_i8(hip(np.zeros((4, 30), np.int8)), hip(np.zeros((8, 30), np.int8)),
                        out_mode=0, path=TILE)


@pytest.mark.parametrize("M,N,K,path", [(394, 768, 768, TILE), (300, 260, 144, TILE), (129, 77, 784, TILE),
                                        (16, 256, 64, SKINNY), (9, 10, 7, NAIVE), (2048, 512, 256, TILE)])
@pytest.mark.parametrize("mode", [_ops.OUT_F32, _ops.OUT_F16])
def test_residual_joins_in_the_epilogue(M, N, K, path, mode):
    """out = (acc * scales + bias) + residual, float32 add, then the store's
    narrowing: x + linear(...) of a transformer block in one kernel."""
    rng = np.random.default_rng(M + N + K + mode)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    got = _ops.qlinear_i8(hip(a), hip(w), a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                          out_mode=mode, path=path, residual=hip(res)).numpy()
    y = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F32) + res
    if mode == _ops.OUT_F16:
        assert np.array_equal(got.view(np.uint16), O.f32_to_f16_bits(y))
    else:
        assert np.array_equal(got, y)


def test_residual_needs_a_float_output():
    a, w = hip(np.zeros((4, 16), np.int8)), hip(np.zeros((4, 16), np.int8))
    with pytest.raises(ValueError):
        _ops.qlinear_i8(a, w, out_mode=_ops.OUT_ACC_I32, residual=hip(np.zeros((4, 4), np.float32)))


@pytest.mark.parametrize("M,N,K,path", [(256, 512, 128, 1), (130, 72, 96, 1), (8, 64, 256, 2), (5, 33, 40, 3)])
def test_fused_join_on_codes(M, N, K, path):
    """qlinear with a join == qlinear to codes, then lq_add_requant_i8 (tile, skinny, naive)."""
    from lucid_amd import _C, _ops
    rng = np.random.default_rng(M + N + K)
    hip = lambda a: L.tensor(a, device="hip")
    a, w = hip(rng.integers(-128, 128, (M, K)).astype(np.int8)), hip(rng.integers(-127, 128, (N, K)).astype(np.int8))
    common = dict(a_zp=5, a_scale=hip(np.float32(0.02)), w_scale=hip((rng.random(N).astype(np.float32) + 0.5) * 1e-3),
                  wsum=_ops.rowsum_i8(w), bias=hip(rng.standard_normal(N).astype(np.float32) * 0.1),
                  out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(0.03)), out_zp=hip(np.float32(-3.0)),
                  out_qmin=-128, out_qmax=127, out_offset=0, path=path)
    first = _ops.qlinear_i8(a, w, **common)
    other = hip(rng.integers(-128, 128, (M, N)).astype(np.int8))
    s2, z2, S, Z = (hip(np.float32(v)) for v in (0.025, 131.0, 0.04, 7.0))
    want = L.Tensor.empty((M, N), L.int8, "hip")
    _C.call("lq_add_requant_i8", first.data_ptr, 0, common["out_scale"].data_ptr, common["out_zp"].data_ptr,
            other.data_ptr, -128, s2.data_ptr, z2.data_ptr, M * N, 1, S.data_ptr, Z.data_ptr, 0, 255, -128,
            want.data_ptr, None)
    fused = _ops.qlinear_i8(a, w, **common, join=dict(q=other, offset=-128, scale=s2, zp=z2, relu=True, out_scale=S,
                                                       out_zp=Z, out_qmin=0, out_qmax=255, out_offset=-128))
    assert np.array_equal(fused.numpy(), want.numpy())


def test_split_k_over_few_tiles_exact():
    """Fewer tiles than block slots and a long K (a late convolution stage as a GEMM): the
    stream-K schedule gives every tile a whole number of workers; exact, like every schedule."""
    M, N, K = 1568, 512, 4608
    rng = np.random.default_rng(99)
    a = rng.integers(-128, 128, (M, K)).astype(np.int8)
    w = rng.integers(-127, 128, (N, K)).astype(np.int8)
    hip = lambda t: L.tensor(t, device="hip")
    acc = _ops.qlinear_i8(hip(a), hip(w), out_mode=_ops.OUT_ACC_I32, path=1, tile_config=5 | 0x200).numpy()
    assert np.array_equal(acc, O.igemm(a, w))
    # and through the automatic choice (which may pick that schedule for this shape)
    assert np.array_equal(_ops.qlinear_i8(hip(a), hip(w), out_mode=_ops.OUT_ACC_I32, path=1).numpy(), acc)


@pytest.mark.parametrize("M,N,K,a_tiles", [(2048, 11008, 256, 32), (300, 1000, 128, 2), (512, 800, 192, 1)])
def test_column_split_between_two_tile_shapes_exact(M, N, K, a_tiles):
    """tile_config bits 16+: the first a_tiles * 256 columns with 256x256 tiles, the rest as a problem
    of its own - every per-column operand (weights, sums, scales, bias, residual, join, output) is offset."""
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-128, 128, (M, K)).astype(np.int8)
    w = rng.integers(-127, 128, (N, K)).astype(np.int8)
    ws = (rng.random(N).astype(np.float32) + 0.5) * 1e-3
    bias = rng.standard_normal(N).astype(np.float32)
    hip = lambda t: L.tensor(t, device="hip")
    da, dw = hip(a), hip(w)
    tc = 1 | (1 << 8) | (a_tiles << 16)
    assert np.array_equal(_ops.qlinear_i8(da, dw, out_mode=_ops.OUT_ACC_I32, path=1, tile_config=tc).numpy(),
                          O.igemm(a, w))
    res = rng.standard_normal((M, N)).astype(np.float32)
    common = dict(a_zp=3, a_scale=hip(np.float32(0.02)), w_scale=hip(ws), wsum=_ops.rowsum_i8(dw), bias=hip(bias))
    y = _ops.qlinear_i8(da, dw, **common, out_mode=_ops.OUT_F32, residual=hip(res), path=1, tile_config=tc).numpy()
    want = _ops.qlinear_i8(da, dw, **common, out_mode=_ops.OUT_F32, residual=hip(res), path=1, tile_config=5 | 0x100)
    assert np.array_equal(y.view(np.uint32), want.numpy().view(np.uint32))
    other = hip(rng.integers(-128, 128, (M, N)).astype(np.int8))
    one = lambda v: hip(np.float32(v))
    jk = dict(out_mode=_ops.OUT_REQUANT_I8, out_scale=one(0.05), out_zp=one(3.0), out_qmin=-128, out_qmax=127,
              join=dict(q=other, offset=-128, scale=one(0.02), zp=one(120.0), relu=True, out_scale=one(0.06),
                        out_zp=one(0.0), out_qmin=0, out_qmax=255, out_offset=-128))
    j1 = _ops.qlinear_i8(da, dw, **common, **jk, path=1, tile_config=tc).numpy()
    j2 = _ops.qlinear_i8(da, dw, **common, **jk, path=1, tile_config=5 | 0x100).numpy()
    assert np.array_equal(j1, j2)


@pytest.mark.parametrize("out_scale", [1.0, 0.5, 3.0, 0.1, 7.3e-4, 1e-30, 1e30])
@pytest.mark.parametrize("relu", [False, True])
def test_requantize_at_ties_near_ties_and_saturation(out_scale, relu):
    """The tile kernel's epilogue avoids the division for most elements (a reciprocal multiply
    with a guard band around the rounding boundaries, the IEEE quotient for the rest).  Power
    of two scales put a large share of the quotients exactly on half-integers (ties to even),
    bias values of +-1 ulp put them just off; tiny and huge scales saturate or zero everything
    and fall outside what the reciprocal route accepts.  Codes must equal the oracle's."""
    rng = np.random.default_rng(int(out_scale * 1000) % 977 + relu)
    M, N, K = 384, 256, 64
    a, w = codes(rng, (M, K), -3, 3), codes(rng, (N, K), -3, 3)
    a_scale = np.float32(0.5)
    w_scale = np.full(N, 0.5, np.float32)
    w_scale[::3] = 0.25
    # bias: zero, +-tiny (pushes exact ties just off the boundary), and halves
    bias = rng.choice(np.array([0.0, 1e-7, -1e-7, 0.5, -0.5, 0.125], np.float32), N).astype(np.float32)
    S, Z = np.float32(out_scale), np.float32(-5.0)
    for mode in (_ops.OUT_REQUANT_I8, _ops.OUT_FAKEQUANT_F32):
        got = _ops.qlinear_i8(hip(a), hip(w), a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                              relu=relu, out_mode=mode, out_scale=hip(S), out_zp=hip(Z), out_qmin=-128,
                              out_qmax=127, out_offset=0, path=TILE).numpy()
        exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, relu=relu, out_mode=mode, out_scale=S, out_zp=Z,
                        out_qmin=-128, out_qmax=127, out_offset=0)
        if mode == _ops.OUT_REQUANT_I8:
            assert np.array_equal(got, exp)
            if out_scale in (1.0, 0.5):  # the case is what it claims to be: many exact ties
                t = (O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, relu=relu, out_mode=O.OUT_F32) / S)
                assert (np.abs(t - np.floor(t) - 0.5) == 0).mean() > 0.02
        else:
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))


def test_fused_join_at_ties_and_with_odd_grids():
    """The fused join on codes through the same guard-band route: power-of-two grids make the
    joined sums land on half-integers; a zero point beyond +-255 switches the route off.  Equal
    to the stand-alone lq_add_requant_i8 (itself checked against the oracle) bit for bit."""
    from lucid_amd import _C
    rng = np.random.default_rng(77)
    M, N, K = 256, 384, 64
    a, w = hip(codes(rng, (M, K), -4, 4)), hip(codes(rng, (N, K), -4, 4))
    for (s1, z1, s2, z2, S, Z) in ((0.5, 0.0, 0.25, 3.0, 1.0, 0.0), (0.5, -3.0, 0.5, 0.0, 2.0, 10.0),
                                    (0.03, 2.0, 0.025, 131.0, 0.04, 7.0), (0.5, 0.0, 0.5, 0.0, 1.0, 300.0)):
        common = dict(a_scale=hip(np.float32(0.5)), w_scale=hip(np.full(N, 0.5, np.float32)),
                      out_mode=_ops.OUT_REQUANT_I8, out_scale=hip(np.float32(s1)), out_zp=hip(np.float32(z1)),
                      out_qmin=-128, out_qmax=127, out_offset=0, path=TILE)
        first = _ops.qlinear_i8(a, w, **common)
        other = hip(codes(rng, (M, N)))
        s2t, z2t, St, Zt = (hip(np.float32(v)) for v in (s2, z2, S, Z))
        want = L.Tensor.empty((M, N), L.int8, "hip")
        _C.call("lq_add_requant_i8", first.data_ptr, 0, common["out_scale"].data_ptr, common["out_zp"].data_ptr,
                other.data_ptr, -128, s2t.data_ptr, z2t.data_ptr, M * N, 0, St.data_ptr, Zt.data_ptr, 0, 255, -128,
                want.data_ptr, None)
        fused = _ops.qlinear_i8(a, w, **common, join=dict(q=other, offset=-128, scale=s2t, zp=z2t, relu=False,
                                                           out_scale=St, out_zp=Zt, out_qmin=0, out_qmax=255,
                                                           out_offset=-128))
        assert np.array_equal(fused.numpy(), want.numpy())
        exp = O.add_requant(first.numpy(), 0, np.float32(s1), np.float32(z1), other.numpy(), -128, np.float32(s2),
                            np.float32(z2), False, np.float32(S), np.float32(Z), 0, 255, -128)
        assert np.array_equal(fused.numpy(), exp.reshape(M, N))


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("zp,qmin,qmax,offset", [
    (0.0, 0, 255, -128),      # unsigned codes stored signed: packed route, XOR
    (128.0, 0, 255, -128),
    (-7.0, -128, 127, 0),     # signed range: shifted by 128 for the packed route
    (-128.0, -128, 127, 0),   # zero point on the lower bound
    (127.0, -128, 127, 0),    # ... on the upper bound: a ReLU leaves one code
    (10.0, 0, 100, -50),      # a storage offset that is no multiple of 128: the general narrowing
    (3.0, 0, 127, 0),         # unsigned subrange stored as is
    (-20.0, 0, 255, -128),    # zero point below the range: a ReLU cannot be folded, every element divides
    (200.0, -128, 127, 0)])   # zero point above the range
def test_requantize_grid_variants_through_the_tile_epilogue(zp, qmin, qmax, offset, relu):
    """The tile epilogue folds the ReLU and the storage form into the clamp bounds where the
    grid allows it and falls back to the plain arithmetic where it does not; both must give
    the oracle's codes.  M is not a multiple of the tile height, so interior and edge tiles
    (vector and scalar stores) both run."""
    rng = np.random.default_rng(int(zp * 2) % 97 + qmax + relu)
    M, N, K = 300, 260, 96
    a, w, a_scale, w_scale, bias, a_zp = _epilogue_case(rng, M, N, K, False, "f32")
    wsum = _ops.rowsum_i8(hip(w))
    y = O.qlinear(a, w, a_zp, a_scale, w_scale, bias=bias, relu=relu, out_mode=O.OUT_F32)
    S, Z = np.float32(np.abs(y).max() / 90 + 1e-6), np.float32(zp)
    for mode in (_ops.OUT_REQUANT_I8, _ops.OUT_FAKEQUANT_F32):
        got = _ops.qlinear_i8(hip(a), hip(w), a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum,
                              bias=hip(bias), relu=relu, out_mode=mode, out_scale=hip(S), out_zp=hip(Z),
                              out_qmin=qmin, out_qmax=qmax, out_offset=offset, path=TILE).numpy()
        exp = O.qlinear(a, w, a_zp, a_scale, w_scale, bias=bias, relu=relu, out_mode=mode, out_scale=S, out_zp=Z,
                        out_qmin=qmin, out_qmax=qmax, out_offset=offset)
        if mode == _ops.OUT_REQUANT_I8:
            assert np.array_equal(got, exp)
            if qmin < zp < qmax:
                assert len(np.unique(got)) > 20  # the case exercises the grid
        else:
            assert np.array_equal(got.view(np.uint32), exp.view(np.uint32))


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("z1,z2,off2,Zj,qmin,qmax,offj", [
    (0.0, 0.0, -128, 0.0, 0, 255, -128),
    (-3.0, 17.0, 0, -9.0, -128, 127, 0),       # every grid signed, partner stored as is
    (5.0, 131.0, -128, 64.0, 0, 255, -128),
    (2.0, 7.5, -128, 3.0, 0, 255, -128),       # partner zero point no integer: the general join
    (2.0, 7.0, -128, 3.0, 0, 100, -50),        # join output with a storage offset that is no multiple of 128
    (2.0, 7.0, -128, -4.0, 0, 255, -128)])     # join zero point below its range: its ReLU is not folded
def test_fused_join_grid_variants(z1, z2, off2, Zj, qmin, qmax, offj, relu):
    """The fused join takes this layer's code minus its zero point from shifted clamp bounds,
    the partner's stored byte in one subtraction, and folds its ReLU and storage form like the
    plain requantize; each has a fallback.  Equal to the oracle's two-step form (requantize,
    then add_requant) on interior and edge tiles."""
    rng = np.random.default_rng(int(z2 * 2) + qmax + relu)
    M, N, K = 300, 260, 64
    a, w = codes(rng, (M, K), -6, 6), codes(rng, (N, K), -6, 6)
    a_scale, w_scale = np.float32(0.11), rng.uniform(0.05, 0.2, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    s1, s2, Sj = np.float32(0.31), np.float32(0.027), np.float32(0.35)
    common = dict(a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias), out_mode=_ops.OUT_REQUANT_I8,
                  out_scale=hip(s1), out_zp=hip(np.float32(z1)), out_qmin=-128, out_qmax=127, out_offset=0,
                  path=TILE)
    lo2, hi2 = (0, 255) if off2 else (-128, 127)
    other = rng.integers(lo2, hi2 + 1, (M, N)).astype(np.int64)
    other_stored = (other + off2).astype(np.int8)
    fused = _ops.qlinear_i8(hip(a), hip(w), **common,
                            join=dict(q=hip(other_stored), offset=off2, scale=hip(s2), zp=hip(np.float32(z2)),
                                      relu=relu, out_scale=hip(Sj), out_zp=hip(np.float32(Zj)), out_qmin=qmin,
                                      out_qmax=qmax, out_offset=offj)).numpy()
    first = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=s1,
                      out_zp=np.float32(z1), out_qmin=-128, out_qmax=127, out_offset=0)
    exp = O.add_requant(first, 0, s1, np.float32(z1), other_stored, off2, s2, np.float32(z2), relu, Sj,
                        np.float32(Zj), qmin, qmax, offj)
    assert np.array_equal(fused, exp.reshape(M, N))
    assert len(np.unique(fused)) > 20


PP_SHAPES = [(256, 256, 128), (300, 260, 192), (513, 1000, 576), (2048, 512, 4096), (1, 16, 64), (700, 130, 64),
             (257, 353, 320), (2048, 1004, 256), (40, 1001, 128)]


@pytest.mark.parametrize("cfg", [13, 14, 16, 21, 22])
@pytest.mark.parametrize("M,N,K", PP_SHAPES)
def test_ping_pong_kernel_exact(cfg, M, N, K):
    """The eight-wavefront kernel (tile_config 13 / 14): accumulators and the float16 epilogue
    against the oracle on full, ragged and tiny shapes (edge tiles, rows read past the end of a
    matrix, widths that rule out the vector and the paired stores)."""
    rng = np.random.default_rng(cfg * 1000 + M + N + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    ad, wd = hip(a), hip(w)
    acc = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=cfg).numpy()
    assert np.array_equal(acc, O.igemm(a, w))
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    got = _ops.qlinear_i8(ad, wd, a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                          out_mode=_ops.OUT_F16, path=TILE, tile_config=cfg).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


@pytest.mark.parametrize("cfg", [13, 14, 16, 21, 22])
@pytest.mark.parametrize("M,N,K", [(512, 704, 256), (300, 260, 128), (129, 1001, 64), (512, 768, 192)])
def test_ping_pong_kernel_every_output_form(cfg, M, N, K):
    """Every epilogue form of the eight-wavefront kernel equals the oracle: an activation zero
    point with the row-sum correction, per-tensor and per-row activation scales, ReLU, float32
    with a residual, requantized codes (both storage forms), fake-quantized float32, and the
    fused join on codes."""
    rng = np.random.default_rng(cfg * 77 + M + N + K)
    a, w = codes(rng, (M, K), -100, 100), codes(rng, (N, K), -100, 100)
    ad, wd = hip(a), hip(w)
    wsum = _ops.rowsum_i8(wd)
    a_zp = 7
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.3).astype(np.float32)
    one = lambda v: hip(np.float32(v))
    for per_row in (False, True):
        a_scale = rng.uniform(0.005, 0.05, M if per_row else 1).astype(np.float32)
        common = dict(a_zp=a_zp, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum, bias=hip(bias), path=TILE,
                      tile_config=cfg)
        ocommon = dict(bias=bias)
        res = rng.standard_normal((M, N)).astype(np.float32)
        for relu in (False, True):
            y = _ops.qlinear_i8(ad, wd, **common, relu=relu, out_mode=_ops.OUT_F32, residual=hip(res)).numpy()
            exp = O.qlinear(a, w, a_zp, a_scale, w_scale, relu=relu, out_mode=O.OUT_F32, **ocommon) + res
            assert np.array_equal(y.view(np.uint32), exp.astype(np.float32).view(np.uint32))
            yf = O.qlinear(a, w, a_zp, a_scale, w_scale, relu=relu, out_mode=O.OUT_F32, **ocommon)
            S = np.float32(np.abs(yf).max() / 100 + 1e-6)
            for (Z, qmin, qmax, off) in ((np.float32(128.0 if not relu else 3.0), 0, 255, -128),
                                         (np.float32(-7.0), -128, 127, 0)):
                kw = dict(out_scale=one(S), out_zp=one(Z), out_qmin=qmin, out_qmax=qmax, out_offset=off)
                okw = dict(out_scale=S, out_zp=Z, out_qmin=qmin, out_qmax=qmax, out_offset=off)
                q = _ops.qlinear_i8(ad, wd, **common, relu=relu, out_mode=_ops.OUT_REQUANT_I8, **kw).numpy()
                assert np.array_equal(q, O.qlinear(a, w, a_zp, a_scale, w_scale, relu=relu,
                                                   out_mode=O.OUT_REQUANT_I8, **ocommon, **okw))
                fq = _ops.qlinear_i8(ad, wd, **common, relu=relu, out_mode=_ops.OUT_FAKEQUANT_F32, **kw).numpy()
                efq = O.qlinear(a, w, a_zp, a_scale, w_scale, relu=relu, out_mode=O.OUT_FAKEQUANT_F32, **ocommon, **okw)
                assert np.array_equal(fq.view(np.uint32), efq.view(np.uint32))
        # the fused join against the two-step form of the oracle
        s1, z1, s2, z2, Sj, Zj = (np.float32(v) for v in (S, 3.0, 0.027, 131.0, S * 1.3, 64.0))
        other = rng.integers(0, 256, (M, N)).astype(np.int64)
        stored = (other - 128).astype(np.int8)
        fused = _ops.qlinear_i8(ad, wd, **common, out_mode=_ops.OUT_REQUANT_I8, out_scale=one(s1), out_zp=one(z1),
                                out_qmin=-128, out_qmax=127, out_offset=0,
                                join=dict(q=hip(stored), offset=-128, scale=one(s2), zp=one(z2), relu=True,
                                          out_scale=one(Sj), out_zp=one(Zj), out_qmin=0, out_qmax=255,
                                          out_offset=-128)).numpy()
        first = O.qlinear(a, w, a_zp, a_scale, w_scale, out_mode=O.OUT_REQUANT_I8, out_scale=s1, out_zp=z1,
                          out_qmin=-128, out_qmax=127, out_offset=0, **ocommon)
        expj = O.add_requant(first, 0, s1, z1, stored, -128, s2, z2, True, Sj, Zj, 0, 255, -128)
        assert np.array_equal(fused, expj.reshape(M, N))


@pytest.mark.parametrize("cfg", [13, 14, 16, 21, 22])
@pytest.mark.parametrize("M,N,K", [(512, 704, 256), (300, 260, 128), (129, 1001, 64), (1576, 3072, 768)])
def test_ping_pong_kernel_gelu_and_kept_range(cfg, M, N, K):
    """GELU in the epilogue and the kept range of what is stored, on the eight-wavefront kernel:
    the bits of the four-wavefront tile kernel (which the stand-alone GELU kernel is tested
    against), with and without a residual, and exactly the minimum and maximum of the result -
    rows and columns of edge tiles past the matrix do not count, a NaN does."""
    from lucid_amd import _C
    rng = np.random.default_rng(cfg * 31 + M + N + K)
    a, w = codes(rng, (M, K), -100, 100), codes(rng, (N, K), -100, 100)
    ad, wd = hip(a), hip(w)
    per_row = cfg != 14
    a_scale = rng.uniform(0.002, 0.01, M if per_row else 1).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.3).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    common = dict(a_zp=5, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=_ops.rowsum_i8(wd), bias=hip(bias),
                  out_mode=_ops.OUT_F32, path=TILE)

    def kept(buf):
        mn, mx = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
        s, z = L.Tensor.empty((), L.float32, "hip"), L.Tensor.empty((), L.float32, "hip")
        _C.call("lq_calc_qparams_from_range", buf.data_ptr, 0, 0, 255, 0, 1e-8, s.data_ptr, z.data_ptr, mn.data_ptr,
                mx.data_ptr, None)
        return float(mn.numpy()), float(mx.numpy())

    for residual in (None, res):
        kw = dict(common, residual=hip(residual) if residual is not None else None)
        rb = L.Tensor.empty((_C.range_buffer_words(),), L.float32, "hip")
        got = _ops.qlinear_i8(ad, wd, **kw, gelu=True, range_buf=rb, tile_config=cfg).numpy()
        assert _C.load().lq_last_tile_config() & 0xff == cfg
        want = _ops.qlinear_i8(ad, wd, **kw, gelu=True, tile_config=5).numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        assert kept(rb) == (float(want.min()), float(want.max()))
        # a kept range without the GELU
        rb2 = L.Tensor.empty((_C.range_buffer_words(),), L.float32, "hip")
        plain = _ops.qlinear_i8(ad, wd, **kw, range_buf=rb2, tile_config=cfg).numpy()
        assert np.array_equal(plain.view(np.uint32), _ops.qlinear_i8(ad, wd, **kw, tile_config=5).numpy().view(np.uint32))
        assert kept(rb2) == (float(plain.min()), float(plain.max()))
    # a NaN in one stored element reaches the range
    bad = res.copy()
    bad[M - 1, N - 1] = np.nan
    rb = L.Tensor.empty((_C.range_buffer_words(),), L.float32, "hip")
    _ops.qlinear_i8(ad, wd, **common, residual=hip(bad), gelu=True, range_buf=rb, tile_config=cfg)
    mn, mx = kept(rb)
    assert np.isnan(mn) and np.isnan(mx)


# ------------------------------------------------------------------ affine weight codes
AFFINE_CASES = [
    # M, N, K, path
    (64, 256, 784, TILE), (300, 260, 144, TILE), (2048, 512, 1024, TILE), (1, 11008, 4096, SKINNY),
    (16, 1024, 4096, SKINNY), (17, 33, 784, SKINNY), (5, 7, 3, NAIVE), (64, 10, 250, NAIVE), (129, 77, 784, 0),
]


@pytest.mark.parametrize("M,N,K,path", AFFINE_CASES)
def test_affine_weight_zero_points_every_output_form(M, N, K, path):
    """Per-channel affine weights (a zero point per weight row): every output form equals the
    oracle's term-by-term sum of (a - za) * (w - zw[n]) bit for bit."""
    rng = np.random.default_rng(M * 5 + N * 11 + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    zw = rng.integers(-128, 128, N).astype(np.int32)
    zw[::7] = 0
    za = int(rng.integers(-128, 128))
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.5).astype(np.float32)
    y = O.qlinear(a, w, za, a_scale, w_scale, bias=bias, relu=True, w_zp=zw)
    S, Z = np.float32(y.max() / 250 + 1e-6), np.float32(2.0)
    ad, wd = hip(a), hip(w)
    dkw = dict(a_zp=za, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=_ops.rowsum_i8(wd), bias=hip(bias),
               relu=True, out_scale=hip(S), out_zp=hip(Z), out_qmin=0, out_qmax=255, out_offset=-128,
               w_zp=hip(zw), path=path)
    okw = dict(bias=bias, relu=True, out_scale=S, out_zp=Z, out_qmin=0, out_qmax=255, out_offset=-128, w_zp=zw)
    for mode in (_ops.OUT_F32, _ops.OUT_F16, _ops.OUT_REQUANT_I8, _ops.OUT_FAKEQUANT_F32):
        got = _ops.qlinear_i8(ad, wd, out_mode=mode, **dkw).numpy()
        exp = O.qlinear(a, w, za, a_scale, w_scale, out_mode=mode, **okw)
        assert np.array_equal(got.view(np.uint8), exp.view(np.uint8)), mode
    # the raw accumulators are the sums a * w: weight zero points cannot apply to them and are refused
    with pytest.raises(ValueError, match="ACC_I32"):
        _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, w_zp=hip(zw), wsum=_ops.rowsum_i8(wd), path=path)
    acc = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=path)
    assert np.array_equal(acc.numpy(), O.igemm(a, w))


def test_affine_weights_with_device_zero_point_residual_and_join():
    """The corrections compose with the other epilogue operands: a zero point that lives on
    the device (dynamic quantization), a float residual, a GELU, and the join on codes."""
    rng = np.random.default_rng(77)
    M, N, K = 70, 96, 320
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    zw = rng.integers(-100, 100, N).astype(np.int32)
    a_scale, w_scale = np.float32(0.02), rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    res = rng.standard_normal((M, N)).astype(np.float32)
    ad, wd = hip(a), hip(w)
    wsum = _ops.rowsum_i8(wd)
    # effective zero point = int(*a_zp_dev) + a_zp = 133 - 128
    got = _ops.qlinear_i8(ad, wd, a_zp=-128, a_zp_dev=hip(np.float32(133.0)), a_scale=hip(a_scale),
                          w_scale=hip(w_scale), wsum=wsum, bias=hip(bias), residual=hip(res), w_zp=hip(zw)).numpy()
    exp = O.qlinear(a, w, 5, a_scale, w_scale, bias=bias, w_zp=zw) + res
    assert np.array_equal(got.view(np.uint32), exp.astype(np.float32).view(np.uint32))
    # the symmetric call with the same weights differs, so w_zp is really applied
    sym = _ops.qlinear_i8(ad, wd, a_zp=5, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum,
                          bias=hip(bias)).numpy()
    assert not np.array_equal(sym + res, got)
    # join on codes: identical to the unfused pair on the affine layer's own codes
    S1, Z1 = hip(np.float32(0.05)), hip(np.float32(120.0))
    other = codes(rng, (M, N))
    join = dict(q=hip(other), offset=-128, scale=hip(np.float32(0.04)), zp=hip(np.float32(131.0)), relu=True,
                out_scale=hip(np.float32(0.06)), out_zp=hip(np.float32(0.0)), out_qmin=0, out_qmax=255,
                out_offset=-128)
    kw = dict(a_zp=5, a_scale=hip(a_scale), w_scale=hip(w_scale), wsum=wsum, bias=hip(bias),
              out_mode=_ops.OUT_REQUANT_I8, out_scale=S1, out_zp=Z1, out_qmin=0, out_qmax=255, out_offset=-128)
    fused_sym = _ops.qlinear_i8(ad, wd, join=join, **kw).numpy()
    fused_aff = _ops.qlinear_i8(ad, wd, join=join, w_zp=hip(zw), **kw).numpy()
    fused_zero = _ops.qlinear_i8(ad, wd, join=join, w_zp=hip(np.zeros(N, np.int32)), **kw).numpy()
    assert np.array_equal(fused_zero, fused_sym)            # the two-pass route with zw = 0 is the one-pass result
    assert not np.array_equal(fused_aff, fused_sym)
    # fused_aff against the oracle composition: layer codes, then add_relu_requant
    c1 = O.qlinear(a, w, 5, a_scale, w_scale, bias=bias, out_mode=O.OUT_REQUANT_I8, out_scale=0.05, out_zp=120.0,
                   out_offset=-128, w_zp=zw)
    exp = O.add_requant(c1, -128, 0.05, 120.0, other, -128, 0.04, 131.0, True, 0.06, 0.0, 0, 255, -128)
    assert np.array_equal(fused_aff, exp)


def test_affine_weights_reject_what_they_cannot_do():
    rng = np.random.default_rng(1)
    a, w = hip(codes(rng, (4, 64))), hip(codes(rng, (8, 64)))
    zw = hip(np.ones(8, np.int32))
    one = hip(np.float32(1.0))
    with pytest.raises(ValueError, match="row sums"):
        _ops.qlinear_i8(a, w, a_scale=one, w_scale=hip(np.ones(8, np.float32)), w_zp=zw)
    with pytest.raises(L.ShapeMismatch):
        _ops.qlinear_i8(a, w, a_scale=one, w_scale=hip(np.ones(8, np.float32)), wsum=_ops.rowsum_i8(w),
                        w_zp=hip(np.ones(7, np.int32)))


def _llm_layer(rng, M, K=4096, N=11008):
    wf = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    mn, mx = O.minmax(wf, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    wq = O.quantize(wf, ws, wz, -128, 127, ch_axis=0)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    x = rng.standard_normal((M, K)).astype(np.float32)
    mn, mx = O.minmax(x, ch_axis=0)
    xs, xz = O.calc_qparams(mn, mx, True, -128, 127, True)
    xq = O.quantize(x, xs, xz, -128, 127, ch_axis=0)
    return xq, xs, wq, ws, bias


def test_headline_shape_on_the_forced_ping_pong_kernel():
    """M=2048, K=4096, N=11008 with tile_config 13 forced: the full grid of 8 x 32 tiles of
    256 x 352 (one per compute unit, the last tile column mostly padding).  float16 output
    against the oracle on rows sampled from every tile row; exact accumulators in full through
    linearity, and a whole tile column (all 2048 rows x the last 96 real columns plus the
    columns of the first tile) against the oracle's integer GEMM."""
    from lucid_amd import _C
    rng = np.random.default_rng(2048)
    M, K, N = 2048, 4096, 11008
    xq, xs, wq, ws, bias = _llm_layer(rng, M)
    xd, wd = hip(xq), hip(wq)
    got = _ops.qlinear_i8(xd, wd, a_scale=hip(xs), w_scale=hip(ws), bias=hip(bias), out_mode=_ops.OUT_F16,
                          path=TILE, tile_config=13 | 0x100).numpy()
    assert _C.load().lq_last_tile_config() == 0x10d
    rows = np.unique(np.concatenate([rng.integers(0, M, 24), np.arange(0, M, 256), np.arange(255, M, 256)]))
    exp = O.qlinear(xq[rows], wq, 0, xs[rows], ws, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got[rows].view(np.uint16), exp.view(np.uint16))
    acc = _ops.qlinear_i8(xd, wd, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=13 | 0x100).numpy()
    cols = np.concatenate([np.arange(0, 352), np.arange(31 * 352, N)])
    assert np.array_equal(acc[:, cols], O.igemm(xq, wq[cols]))
    xa, xb = codes(rng, (M, K), -60, 60), codes(rng, (M, K), -60, 60)
    f = lambda t: _ops.qlinear_i8(hip(t), wd, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=13 | 0x100).numpy()
    assert np.array_equal(f(xa) + f(xb), f((xa + xb).astype(np.int8)))


def test_first_call_under_capture_gets_the_ping_pong_kernel():
    """The tuner may not time candidates on a stream that is being captured; the size rule it
    falls back on must then give a large plain GEMM the eight-wavefront kernel (256 x 352 tiles
    when they fit the 256 compute units better, 256 x 256 otherwise), not the four-wavefront
    128 x 256 shape."""
    from lucid_amd import _C
    rng = np.random.default_rng(5)
    for (M, K, N), want in (((2048, 4096, 11008), 0x10d), ((2048, 1024, 8192), 0x10e), ((4096, 576, 11008 - 352), 0x10d)):
        a, w = codes(rng, (M, K)), codes(rng, (N, K))
        ad, wd = hip(a), hip(w)
        out = L.Tensor.empty((M, N), L.int32, "hip")
        with L.graph.capture() as g:
            _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, out=out)
            cfg = _C.load().lq_last_tile_config()
        assert cfg == want, hex(cfg)
        g.replay()
        _C.call("lq_sync", None)
        rows = rng.integers(0, M, 16)
        assert np.array_equal(out.numpy()[rows], O.igemm(a[rows], w))
        g.destroy()


def test_tuning_choices_export_and_import():
    """lq_tune_export / lq_tune_import: a shape the tuner has timed appears in the exported text;
    an imported line decides a shape this process has never run, without any timing (the
    imported choice is what lq_last_tile_config reports), and the result is unchanged."""
    import ctypes as C
    from lucid_amd import _C
    lib = _C.load()
    rng = np.random.default_rng(9)
    M, K, N = 640, 512, 768
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    ad, wd = hip(a), hip(w)
    _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32)          # tuned here (0.5 GOP is the tuner's floor)
    chosen = lib.lq_last_tile_config()
    need = C.c_size_t()
    _C.call("lq_tune_export", None, 0, C.byref(need))
    buf = C.create_string_buffer(need.value)
    _C.call("lq_tune_export", buf, need.value, C.byref(need))
    lines = [ln for ln in buf.value.decode().splitlines() if ln.startswith("lq-tune-1 ")]
    mine = [ln for ln in lines if ln.split()[1:4] == [str(M), str(N), str(K)]]
    # the table keeps the tuner's candidate value (schedule 0 = one block per tile), the launch reports it resolved
    assert len(mine) == 1 and int(mine[0].split()[-1]) & 0xff == chosen & 0xff
    with pytest.raises(ValueError):
        _C.call("lq_tune_export", buf, 1, C.byref(need))
    # the same key with other extents and a shape the tuner would not pick first: 64 x 64 tiles
    M2, N2 = 648, 776
    fields = mine[0].split()
    fields[1:4] = [str(M2), str(N2), str(K)]
    fields[-1] = str(9 | 0x100)
    taken = C.c_int()
    _C.call("lq_tune_import", ("# a comment\n" + " ".join(fields) + "\n").encode(), C.byref(taken))
    assert taken.value == 1
    a2, w2 = codes(rng, (M2, K)), codes(rng, (N2, K))
    acc = _ops.qlinear_i8(hip(a2), hip(w2), out_mode=_ops.OUT_ACC_I32).numpy()
    assert lib.lq_last_tile_config() == (9 | 0x100)
    assert np.array_equal(acc, O.igemm(a2, w2))
    with pytest.raises(ValueError):
        _C.call("lq_tune_import", b"lq-tune-1 1 2 3\n", None)


def test_first_calls_from_two_threads():
    """Two threads of a fresh process make their first launches at once (kernel attributes, the
    padding table and the tuner's table are set up on first use): both get right results."""
    import os, subprocess, sys, textwrap
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    script = textwrap.dedent("""
        import sys, threading
        import numpy as np
        sys.path.insert(0, %r)
        import lucid_amd as L
        from lucid_amd import _C, _ops
        import oracle as O
        _C.init(0)
        rng = np.random.default_rng(3)
        M, K, N = 512, 256, 704
        a = rng.integers(-128, 128, (M, K)).astype(np.int8)
        w = rng.integers(-128, 128, (N, K)).astype(np.int8)
        want = O.igemm(a, w)
        ad, wd = L.tensor(a, device="hip"), L.tensor(w, device="hip")
        go, bad = threading.Barrier(2), []
        def run(cfg):
            go.wait()
            for _ in range(3):
                got = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=_ops.PATH_TILE, tile_config=cfg).numpy()
                if not np.array_equal(got, want):
                    bad.append(cfg)
        ts = [threading.Thread(target=run, args=(c,)) for c in (13, 13)]
        [t.start() for t in ts]; [t.join() for t in ts]
        print("BAD" if bad else "OK", flush=True)
    """ % root)
    r = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout + r.stderr


@pytest.mark.parametrize("M,N,K", [(256, 352, 1024), (300, 260, 256), (513, 1000, 384), (2048, 704, 4096), (40, 1001, 512),
                                   (2048, 11008, 256)])
def test_one_wavefront_per_simd_kernel_exact(M, N, K):
    """tile_config 17 (four wavefronts with the whole register file each, MFMAs from inline
    assembly): accumulators and the float16 epilogue against the oracle on full, ragged and edge
    shapes, and the shapes it is not built for are refused."""
    rng = np.random.default_rng(17000 + M + N + K)
    a, w = codes(rng, (M, K)), codes(rng, (N, K))
    ad, wd = hip(a), hip(w)
    acc = _ops.qlinear_i8(ad, wd, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=17).numpy()
    assert np.array_equal(acc, O.igemm(a, w))
    a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
    w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.02).astype(np.float16)
    got = _ops.qlinear_i8(ad, wd, a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                          out_mode=_ops.OUT_F16, path=TILE, tile_config=17).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))
    # with a ReLU (the general epilogue) as well
    got = _ops.qlinear_i8(ad, wd, a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias), relu=True,
                          out_mode=_ops.OUT_F16, path=TILE, tile_config=17).numpy()
    exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, relu=True, out_mode=O.OUT_F16)
    assert np.array_equal(got.view(np.uint16), exp.view(np.uint16))


def test_one_wavefront_per_simd_kernel_refusals():
    rng = np.random.default_rng(1)
    a, w = hip(codes(rng, (256, 192))), hip(codes(rng, (256, 192)))
    with pytest.raises(L.ShapeMismatch, match="multiple of 128"):
        _ops.qlinear_i8(a, w, out_mode=_ops.OUT_ACC_I32, path=TILE, tile_config=17)
    a, w = hip(codes(rng, (256, 256))), hip(codes(rng, (256, 256)))
    one = hip(np.ones(256, np.float32))
    with pytest.raises(NotImplementedError, match="output mode"):
        _ops.qlinear_i8(a, w, a_scale=one, w_scale=one, out_mode=_ops.OUT_F32, path=TILE, tile_config=17)


def test_matrix_edges_on_tile_boundaries_take_the_fast_epilogue_and_stay_exact():
    """The float16 / float32 epilogue of the large-GEMM kernels skips whole 16 x 16 tiles past the
    end of the matrix (N = 11008 ends 96 columns into its last 352-wide tile; M = 12608 ends 64
    rows into its last 256-high one): results against the oracle where M and N end on, next to
    and off a tile boundary."""
    rng = np.random.default_rng(33)
    K = 128
    for M, N in ((256 + 64, 352 + 96), (256 + 64, 352 + 100), (256 + 70, 352 + 96), (512 + 16, 704 + 176 + 16), (272, 256 + 48)):
        a, w = codes(rng, (M, K)), codes(rng, (N, K))
        a_scale = rng.uniform(0.005, 0.05, M).astype(np.float32)
        w_scale = rng.uniform(0.0005, 0.004, N).astype(np.float32)
        bias = (rng.standard_normal(N) * 0.02).astype(np.float32)
        for cfg in (13, 14, 16):
            for mode, omode, dt in ((_ops.OUT_F16, O.OUT_F16, np.uint16), (_ops.OUT_F32, O.OUT_F32, np.uint32)):
                got = _ops.qlinear_i8(hip(a), hip(w), a_scale=hip(a_scale), w_scale=hip(w_scale), bias=hip(bias),
                                      out_mode=mode, path=TILE, tile_config=cfg).numpy()
                exp = O.qlinear(a, w, 0, a_scale, w_scale, bias=bias, out_mode=omode)
                assert np.array_equal(got.view(dt), exp.view(dt)), (M, N, cfg, mode)
