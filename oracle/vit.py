"""CPU restatement of Lucid's dynamic-quantized ViT forward (numpy float32 +
the C oracle for the quantized Linears).

TEST INFRASTRUCTURE ONLY, like the rest of ``oracle/``.

Each step cites the reference it follows:

* patch embedding   ``lucid/models/vision/vit/_model.py:62-69`` (Conv2d, stride = kernel)
* tokens            ``_model.py:452-454`` (cat class token, add position table)
* LayerNorm         ``lucid/_C/backend/cpu/Norm.cpp:35-65``
* attention         ``_model.py:137-158``; ``CpuBackend.h:7697-7722`` (scale*QK^T,
                    max-subtracted softmax, weights @ V)
* GELU              ``lucid/nn/functional/activations.py:219`` (erf form)
* dynamic Linear    ``lucid/nn/quantized/dynamic/linear.py:84-99`` in its exact
                    integer formulation (``oracle.qlinear``)

PARITY UNPINNED at the bit level for the float32 steps: the reference sums
through Accelerate (vDSP / cblas) whose accumulation order is not published, so
only tolerance-level agreement is claimed; the float64 evaluation in
``tests/test_oracle_vit.py`` pins each step's formula.
"""

from __future__ import annotations

import math

import numpy as np

import oracle as O

try:  # erf without scipy is fine too, but scipy is in the image
    from scipy.special import erf as _erf
except Exception:  # pragma: no cover
    _erf = np.vectorize(math.erf)


def layer_norm(x, gamma, beta, eps):
    x = np.asarray(x, np.float32)
    n = np.float32(x.shape[-1])
    mean = (x.sum(-1, keepdims=True, dtype=np.float32) / n).astype(np.float32)
    c = (x - mean).astype(np.float32)
    var = ((c * c).sum(-1, keepdims=True, dtype=np.float32) / n).astype(np.float32)
    rstd = (np.float32(1.0) / np.sqrt(var + np.float32(eps))).astype(np.float32)
    return ((c * rstd) * np.asarray(gamma, np.float32) + np.asarray(beta, np.float32)).astype(np.float32)


def gelu(x):
    x = np.asarray(x, np.float32)
    return ((np.float32(0.5) * x) *
            (np.float32(1.0) + _erf(x * np.float32(0.70710678118654752440)).astype(np.float32))).astype(np.float32)


def attention_qkv(qkv, heads):
    """qkv (B, T, 3*H*D) packed as (B, T, 3, H, D) -> (B, T, H*D)."""
    qkv = np.asarray(qkv, np.float32)
    B, T, C3 = qkv.shape
    D = C3 // (3 * heads)
    q, k, v = np.transpose(qkv.reshape(B, T, 3, heads, D), (2, 0, 3, 1, 4))  # each (B, H, T, D)
    s = np.matmul(q * np.float32(1.0 / math.sqrt(D)), np.transpose(k, (0, 1, 3, 2))).astype(np.float32)
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s).astype(np.float32)
    w = (e * (np.float32(1.0) / e.sum(-1, keepdims=True, dtype=np.float32))).astype(np.float32)
    o = np.matmul(w, v).astype(np.float32)
    return np.ascontiguousarray(np.transpose(o, (0, 2, 1, 3)).reshape(B, T, heads * D))


def patch_rows(img, patch):
    """(B, C, H, W) -> (B * gh * gw, C * p * p), columns in (c, ph, pw) order."""
    img = np.asarray(img, np.float32)
    B, C, H, W = img.shape
    gh, gw = H // patch, W // patch
    x = img.reshape(B, C, gh, patch, gw, patch)
    return np.ascontiguousarray(np.transpose(x, (0, 2, 4, 1, 3, 5)).reshape(B * gh * gw, C * patch * patch))


def quantize_weight(w):
    """Per-output-channel symmetric qint8 (``nn/quantized/_utils.py:27-55``)."""
    mn, mx = O.minmax(w, ch_axis=0)
    s, z = O.calc_qparams(mn, mx, True, -128, 127, True)
    return O.quantize(w, s, z, -128, 127, ch_axis=0), s


def dynamic_linear(x, wq, w_scale, bias):
    """``nnqd.Linear.forward``: runtime per-tensor affine quint8 activation,
    int8 GEMM, float32 output.  Codes are carried as code - 128."""
    x = np.asarray(x, np.float32)
    lead, K = x.shape[:-1], x.shape[-1]
    x2 = x.reshape(-1, K)
    mn, mx = O.minmax(x2)
    s, z = O.calc_qparams(mn, mx, False, 0, 255, False)
    xq = O.quantize(x2, s, z, 0, 255, code_offset=-128)
    y = O.qlinear(xq, wq, int(z[0]) - 128, s, w_scale, bias=bias, out_mode=O.OUT_F32)
    return y.reshape(*lead, wq.shape[0])


def vit_forward(p, images, cfg, stages=None):
    """Logits of the dynamic-quantized ViT for float32 NCHW ``images``.  When
    ``stages`` is a dict, intermediate activations are stored into it."""
    d, heads, ps = cfg["dim"], cfg["heads"], cfg["patch"]
    B = images.shape[0]
    rows = patch_rows(images, ps)
    emb = (rows @ p["patch.weight"].reshape(d, -1).T + p["patch.bias"]).astype(np.float32)
    tok = np.concatenate([np.broadcast_to(p["cls"], (B, 1, d)), emb.reshape(B, -1, d)], axis=1)
    x = (tok + p["pos"][None]).astype(np.float32)
    if stages is not None:
        stages["tokens"] = x.copy()
    qw = {}
    for name in ("qkv", "proj", "fc1", "fc2"):
        for i in range(cfg["depth"]):
            qw[f"blocks.{i}.{name}"] = quantize_weight(p[f"blocks.{i}.{name}.weight"])
    qw["head"] = quantize_weight(p["head.weight"])
    for i in range(cfg["depth"]):
        b = f"blocks.{i}."
        h = layer_norm(x, p[b + "norm1.weight"], p[b + "norm1.bias"], 1e-6)
        qkv = dynamic_linear(h, *qw[b + "qkv"], p[b + "qkv.bias"])
        a = attention_qkv(qkv, heads)
        x = (x + dynamic_linear(a, *qw[b + "proj"], p[b + "proj.bias"])).astype(np.float32)
        h = layer_norm(x, p[b + "norm2.weight"], p[b + "norm2.bias"], 1e-6)
        h = gelu(dynamic_linear(h, *qw[b + "fc1"], p[b + "fc1.bias"]))
        x = (x + dynamic_linear(h, *qw[b + "fc2"], p[b + "fc2.bias"])).astype(np.float32)
        if stages is not None:
            stages[f"block{i}"] = x.copy()
    x = layer_norm(x, p["norm.weight"], p["norm.bias"], 1e-6)
    return dynamic_linear(x[:, 0], *qw["head"], p["head.bias"])
