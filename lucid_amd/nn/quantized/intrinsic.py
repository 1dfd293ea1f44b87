"""Fused quantized layers (``lucid/nn/quantized/intrinsic.py``): the ReLU runs
before the output requantize, inside the kernel epilogue."""

from __future__ import annotations

from .conv import Conv1d, Conv2d, Conv3d
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


def _unwrap_fused(mod):
    """The weighted layer of a fused float pair, carrying the pair's qconfig and observer."""
    if not hasattr(mod, "__getitem__"):
        return mod
    inner = mod[0]
    inner.qconfig = mod.qconfig
    inner.activation_post_process = mod.activation_post_process
    return inner


class ConvReLU1d(Conv1d):
    """Quantized ``Conv1d`` + ``ReLU`` (``intrinsic.py:141-240``)."""

    _fused_relu = True

    @classmethod
    def from_float(cls, mod) -> "ConvReLU1d":
        return super().from_float(_unwrap_fused(mod))


class ConvReLU3d(Conv3d):
    """Quantized ``Conv3d`` + ``ReLU`` (``intrinsic.py:344-440``)."""

    _fused_relu = True

    @classmethod
    def from_float(cls, mod) -> "ConvReLU3d":
        return super().from_float(_unwrap_fused(mod))
