"""The float32 steps of the ViT restatement (oracle/vit.py) against float64
evaluations of the same formulas and against torch's own operators; CPU only."""

import math

import numpy as np
import pytest
import torch

import oracle.vit as V


def rel(a, b):
    return float(np.max(np.abs(a.astype(np.float64) - b)) / max(1e-30, np.max(np.abs(b))))


@pytest.mark.parametrize("shape", [(7, 768), (3, 5, 64), (1, 1)])
def test_layer_norm_formula(shape):
    rng = np.random.default_rng(sum(shape))
    x = (rng.standard_normal(shape) * 3 + 1).astype(np.float32)
    g = rng.standard_normal(shape[-1]).astype(np.float32)
    b = rng.standard_normal(shape[-1]).astype(np.float32)
    x64 = x.astype(np.float64)
    mean = x64.mean(-1, keepdims=True)
    var = ((x64 - mean) ** 2).mean(-1, keepdims=True)  # biased, as Norm.cpp:57
    ref = (x64 - mean) / np.sqrt(var + 1e-6) * g + b
    assert rel(V.layer_norm(x, g, b, 1e-6), ref) < 1e-5
    t = torch.nn.functional.layer_norm(torch.from_numpy(x), (shape[-1],), torch.from_numpy(g),
                                       torch.from_numpy(b), 1e-6).numpy()
    assert rel(V.layer_norm(x, g, b, 1e-6), t.astype(np.float64)) < 1e-5


def test_gelu_is_the_erf_form():
    x = np.linspace(-6, 6, 4001).astype(np.float32)
    ref = np.array([0.5 * v * (1 + math.erf(v / math.sqrt(2))) for v in x.astype(np.float64)])
    assert rel(V.gelu(x), ref) < 1e-6
    t = torch.nn.functional.gelu(torch.from_numpy(x)).numpy()
    assert rel(V.gelu(x), t.astype(np.float64)) < 1e-6
    # the tanh approximation differs by far more than this tolerance
    tanh = torch.nn.functional.gelu(torch.from_numpy(x), approximate="tanh").numpy()
    assert rel(tanh, ref) > 1e-5


@pytest.mark.parametrize("B,T,H", [(2, 197, 12), (1, 5, 2), (3, 16, 1)])
def test_attention_matches_torch_sdpa_on_the_packed_layout(B, T, H):
    D = 64
    rng = np.random.default_rng(B * 100 + T + H)
    qkv = rng.standard_normal((B, T, 3 * H * D)).astype(np.float32)
    t = torch.from_numpy(qkv).reshape(B, T, 3, H, D).permute(2, 0, 3, 1, 4)  # vit/_model.py:138
    ref = torch.nn.functional.scaled_dot_product_attention(t[0].double(), t[1].double(), t[2].double())
    ref = ref.permute(0, 2, 1, 3).reshape(B, T, H * D).numpy()
    assert rel(V.attention_qkv(qkv, H), ref) < 1e-5


def test_patch_rows_times_flat_weight_is_the_strided_convolution():
    rng = np.random.default_rng(5)
    img = rng.standard_normal((2, 3, 32, 48)).astype(np.float32)
    w = rng.standard_normal((10, 3, 16, 16)).astype(np.float32)
    b = rng.standard_normal(10).astype(np.float32)
    ref = torch.nn.functional.conv2d(torch.from_numpy(img).double(), torch.from_numpy(w).double(),
                                     torch.from_numpy(b).double(), stride=16)
    ref = ref.reshape(2, 10, -1).permute(0, 2, 1).reshape(-1, 10).numpy()  # vit/_model.py:69
    got = V.patch_rows(img, 16).astype(np.float64) @ w.reshape(10, -1).T.astype(np.float64) + b
    assert rel(got.astype(np.float32), ref) < 1e-6


def test_dynamic_linear_is_within_a_code_of_the_float_formulation():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((40, 96)).astype(np.float32)
    w = (rng.standard_normal((24, 96)) * 0.05).astype(np.float32)
    b = rng.standard_normal(24).astype(np.float32)
    wq, ws = V.quantize_weight(w)
    y = V.dynamic_linear(x, wq, ws, b)
    # float formulation of dynamic/linear.py:84-99: fake-quantized x times dequantized W
    s = (x.max() - min(x.min(), 0)) / 255.0
    z = np.clip(0 - np.rint(min(x.min(), 0) / s), 0, 255)
    xfq = (np.clip(np.rint(x / s) + z, 0, 255) - z) * s
    ref = xfq.astype(np.float64) @ (wq.astype(np.float64) * ws[:, None]).T + b
    assert rel(y, ref) < 1e-4
