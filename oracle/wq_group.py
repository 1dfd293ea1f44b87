"""CPU restatement of the group-wise weight-only path
(``lucid/quantization/_qgemm.py:69-320``), numpy float32.

TEST INFRASTRUCTURE ONLY, like the rest of ``oracle/``.

Lucid delegates these three operators to MLX (``mlx>=0.31``, ``pyproject.toml:17``;
``lucid/_C/ops/quantized/QuantizedMatmul.cpp:47-115`` calls ``mlx::core::quantize`` /
``dequantize`` / ``quantized_matmul``), and MLX is not part of the Lucid checkout.  This
follows the documented contract that ``_qgemm.py:84-97,167-171`` restates:

    s = (max - min) / (2^bits - 1), beta = min, c = clip(round((w - beta) / s), 0, 2^bits - 1)
    w_hat = c * s + beta,   y = x @ w_hat.T

PARITY UNPINNED against MLX's own bits (its kernel may choose the scale's sign and the
anchoring edge differently); pinned here are the contract's properties and the reference's
own tests for this path (``test_real_gemm.py:29-94``): reconstruction within half a step,
packed shapes and densities, accuracy bounds of the Linear (2 % at 8 bits, 15 % at 4), and
agreement of the fused matmul with the dequantize path to 1e-3.
"""

from __future__ import annotations

import numpy as np


def quantize(w, group_size=64, bits=8):
    w = np.asarray(w, np.float32)
    N, K = w.shape
    g = w.reshape(N, K // group_size, group_size)
    lo = g.min(-1, keepdims=True)
    hi = g.max(-1, keepdims=True)
    nmax = np.float32((1 << bits) - 1)
    s = np.maximum(((hi - lo) / nmax).astype(np.float32), np.float32(1e-7))
    c = np.clip(np.rint(((g - lo) / s).astype(np.float32)), 0, nmax).astype(np.uint32).reshape(N, K)
    per = 32 // bits
    shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    packed = (c.reshape(N, K // per, per) << shifts).sum(-1, dtype=np.uint64).astype(np.uint32)
    return packed.view(np.int32), s.reshape(N, -1), lo.reshape(N, -1).astype(np.float32)


def unpack(packed, bits):
    p = np.asarray(packed).view(np.uint32)
    per = 32 // bits
    shifts = (np.arange(per, dtype=np.uint32) * np.uint32(bits))
    return ((p[..., None] >> shifts) & np.uint32((1 << bits) - 1)).reshape(p.shape[0], -1)


def dequantize(packed, scales, biases, group_size=64, bits=8):
    c = unpack(packed, bits).astype(np.float32)
    s = np.repeat(np.asarray(scales, np.float32), group_size, axis=1)
    b = np.repeat(np.asarray(biases, np.float32), group_size, axis=1)
    return (c * s + b).astype(np.float32)


def matmul(x, packed, scales, biases, group_size=64, bits=8):
    w = dequantize(packed, scales, biases, group_size, bits)
    return (np.asarray(x, np.float64) @ w.astype(np.float64).T).astype(np.float32)
