"""Fused quantized layers (``lucid/nn/quantized/intrinsic.py``): the ReLU runs
before the output requantize, inside the kernel epilogue."""

from __future__ import annotations

from .conv import Conv2d
from .linear import Linear


class LinearReLU(Linear):
    """Quantized ``Linear`` + ``ReLU`` (``intrinsic.py:23-37,131-138``)."""

    _fused_relu = True

    def _activation(self, y):
        from .. import relu
        return relu(y)

    @classmethod
    def from_float(cls, mod) -> "LinearReLU":
        # an nni.LinearReLU is a Sequential(Linear, ReLU) that carries the qconfig
        # and the activation observer of the fused pair
        # (a QAT LinearReLU is already a single weighted layer: intrinsic.py:23-37)
        if not hasattr(mod, "__getitem__"):
            return super().from_float(mod)
        inner = mod[0]
        inner.qconfig = mod.qconfig
        inner.activation_post_process = mod.activation_post_process
        return super().from_float(inner)


class ConvReLU2d(Conv2d):
    """Quantized ``Conv2d`` + ``ReLU`` (``intrinsic.py:334-341``)."""

    _fused_relu = True

    def _activation(self, y):
        from .. import relu
        return relu(y)

    @classmethod
    def from_float(cls, mod) -> "ConvReLU2d":
        if not hasattr(mod, "__getitem__"):  # a QAT ConvReLU2d is a single weighted layer
            return super().from_float(mod)
        inner = mod[0]
        inner.qconfig = mod.qconfig
        inner.activation_post_process = mod.activation_post_process
        return super().from_float(inner)
