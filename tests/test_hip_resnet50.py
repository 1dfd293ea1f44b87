"""End-to-end GPU test of the int8 static-quantized ResNet-50 workload
(workloads.QResNet50) against the oracle's integer formulation, layer by
layer, at a reduced resolution the oracle finishes in seconds."""

import numpy as np
import pytest

import lucid_amd as L
import oracle as O
import workloads as W

pytestmark = pytest.mark.gpu


def _qp(rng_range):
    s, z = O.calc_qparams(np.float32(rng_range[0]), np.float32(rng_range[1]), False, 0, 255, False)
    return np.float32(s[0]), np.float32(z[0])


def _wq(w):
    mn, mx = O.minmax(w, ch_axis=0)
    ws, wz = O.calc_qparams(mn, mx, True, -128, 127, True)
    return O.quantize(w, ws, wz, -128, 127, ch_axis=0), ws


def _oracle_forward(params, calib, x):
    specs = {c[0]: c for c in W.resnet50_convs()}
    s, z = _qp(calib["input"])
    q = O.quantize(x.transpose(0, 2, 3, 1), s, z, 0, 255, code_offset=-128)
    grid = (s, z)

    def conv(name, q, grid):
        _n, _ci, _co, k, st, p, relu = specs[name]
        w, b = params[name]
        wq, ws = _wq(w)
        so, zo = _qp(calib[name])
        out = O.qconv2d(q, wq.transpose(0, 2, 3, 1), int(grid[1]) - 128, grid[0], ws,
                        stride=(st, st), pad=(p, p, p, p), bias=b, relu=relu,
                        out_mode=O.OUT_REQUANT_I8, out_scale=so, out_zp=zo, out_offset=-128)
        return out, (so, zo)

    q, grid = conv("conv1", q, grid)
    q = O.maxpool2d_nhwc_i8(q, (3, 3), (2, 2), (1, 1))
    for si, (_pl, blocks, _st) in enumerate(W.STAGES, start=1):
        for b in range(blocks):
            p = f"layer{si}.{b}"
            idt, gi = conv(f"{p}.downsample", q, grid) if b == 0 else (q, grid)
            o, go = conv(f"{p}.conv1", q, grid)
            o, go = conv(f"{p}.conv2", o, go)
            o, go = conv(f"{p}.conv3", o, go)
            sa, za = _qp(calib[f"{p}.add"])
            q = O.add_requant(o, -128, go[0], go[1], idt, -128, gi[0], gi[1], True, sa, za, 0, 255,
                              -128)
            grid = (sa, za)
    return q, grid


@pytest.fixture(scope="module")
def model_and_params():
    params = W.resnet50_float_params(seed=0)
    calib = W.load_calibration()
    return W.QResNet50(params, calib), params, calib


def test_structure(model_and_params):
    import lucid_amd.nn.quantized as nnq
    model, _, _ = model_and_params
    convs = [m for m in model.modules() if isinstance(m, nnq.Conv2d)]
    assert len(convs) == 53
    assert sum(isinstance(m, nnq.ConvReLU2d) for m in convs) == 33   # stem + conv1/conv2 of 16 blocks
    assert all(m.weight_int8.dtype is L.int8 for m in convs)
    assert sum(isinstance(m, nnq.QFunctional) for m in model.modules()) == 16
    assert abs(W.resnet50_conv_gmacs(1) - 4.089) < 0.01


def test_trunk_codes_bit_exact_and_logits_close(model_and_params):
    model, params, calib = model_and_params
    rng = np.random.default_rng(11)
    x = rng.uniform(0, 1, (2, 3, 64, 64)).astype(np.float32)
    xd = L.tensor(x, device="hip")
    t = model.blocks(model.maxpool(model.conv1(model.quant(xd))))
    q_exp, grid = _oracle_forward(params, calib, x)
    assert t.shape == (2, 2048, 2, 2) and t._grid.layout == "nhwc"
    assert np.array_equal(t._grid.codes.numpy(), q_exp)
    assert np.float32(t._grid.scale.item()) == grid[0] and t._grid.zero_point.item() == grid[1]
    # float view of the trunk output is Lucid's float-carried activation (NCHW)
    fv = O.dequantize(q_exp, grid[0], grid[1], code_offset=-128).transpose(0, 3, 1, 2)
    assert np.array_equal(t.numpy().view(np.uint32), np.ascontiguousarray(fv).view(np.uint32))

    # classifier: global average pool leaves the grid, the Linear runs Lucid's
    # float formulation -> tolerance-level agreement (its sum order is unpinned)
    y = model(xd).numpy()
    pooled = fv.reshape(2, 2048, -1).astype(np.float64).mean(-1).astype(np.float32)
    got_pool = model.avgpool(t).numpy().reshape(2, 2048)
    assert np.allclose(got_pool, pooled, rtol=1e-6, atol=1e-6)
    wfc, bfc = params["fc"]
    wq, ws = _wq(wfc)
    sf, zf = _qp(calib["fc"])
    ref = O.linear_faithful(got_pool, wq, ws, np.zeros(1000, np.float32), bias=bfc,
                            fq=(sf, zf, 0, 255))
    assert y.shape == (2, 1000)
    assert np.abs(y - ref).max() <= sf * 1.001          # at most one grid step, on rounding ties
    assert (y != ref).mean() < 0.02


def test_full_size_batch_runs_and_is_deterministic(model_and_params):
    model, _, _ = model_and_params
    rng = np.random.default_rng(12)
    x = L.tensor(rng.uniform(0, 1, (32, 3, 224, 224)).astype(np.float32), device="hip")
    y1 = model(x).numpy()
    y2 = model(x).numpy()
    assert y1.shape == (32, 1000) and np.isfinite(y1).all()
    assert np.array_equal(y1, y2)
    assert np.unique(y1).size > 16      # the logits use the grid, not a collapsed range
