"""Conv + BatchNorm folding for inference
(``lucid/nn/utils/fusion.py:31-139``).

``W' = W * gamma / sqrt(var + eps)`` per output channel and
``b' = (b - mean) * gamma / sqrt(var + eps) + beta``, in float32 and in the
reference's operation order.  A one-time host-side step on the float
parameters (they are host tensors until the model is quantized), so it is
plain numpy.
"""

from __future__ import annotations

import copy

import numpy as np

from ... import _tensor as T


def fuse_conv_bn_eval(conv, bn):
    """Return a copy of ``conv`` with ``bn``'s inference-time affine folded in."""
    from .. import BatchNorm1d, BatchNorm2d, BatchNorm3d, Conv1d, Conv2d, Conv3d

    if not isinstance(conv, (Conv1d, Conv2d, Conv3d)):
        raise TypeError(f"fuse_conv_bn_eval: conv must be Conv1d/2d/3d, got {type(conv).__name__}")
    if not isinstance(bn, (BatchNorm1d, BatchNorm2d, BatchNorm3d)):
        raise TypeError(f"fuse_conv_bn_eval: bn must be BatchNorm1d/2d/3d, got {type(bn).__name__}")
    fused = copy.deepcopy(conv)
    eps = np.float32(bn.eps)
    mean = bn.running_mean.numpy().astype(np.float32)
    var = bn.running_var.numpy().astype(np.float32)
    affine = getattr(bn, "affine", True)
    gamma = bn.weight.numpy().astype(np.float32) if affine and bn.weight is not None else None
    beta = bn.bias.numpy().astype(np.float32) if affine and bn.bias is not None else None
    inv_std = np.float32(1.0) / np.sqrt(var + eps)
    scale = inv_std if gamma is None else gamma * inv_std
    weight = fused.weight.numpy().astype(np.float32)
    new_weight = weight * scale.reshape(-1, *([1] * (weight.ndim - 1)))
    old_bias = (fused.bias.numpy().astype(np.float32) if fused.bias is not None
                else np.zeros(weight.shape[0], np.float32))
    new_bias = (old_bias - mean) * scale
    if beta is not None:
        new_bias = new_bias + beta
    dev = fused.weight.device
    fused.register_buffer("weight", T.tensor(new_weight.astype(np.float32), device=dev))
    fused.register_buffer("bias", T.tensor(new_bias.astype(np.float32), device=dev))
    return fused
