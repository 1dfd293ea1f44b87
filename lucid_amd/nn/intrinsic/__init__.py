"""Fused float marker modules (``lucid/nn/intrinsic/modules.py``): a
``Sequential`` whose type tells ``convert`` to install the fused quantized
layer (ReLU before the output requantize)."""

from __future__ import annotations

from ..module import Module


class _Fused(Module):
    def __init__(self, *mods) -> None:
        super().__init__()
        for i, m in enumerate(mods):
            self._modules[str(i)] = m

    def __getitem__(self, i):
        return list(self._modules.values())[i]

    def forward(self, x):
        for m in self._modules.values():
            x = m(x)
        return x


class LinearReLU(_Fused):
    """``Linear`` followed by ``ReLU``."""


class ConvReLU2d(_Fused):
    """``Conv2d`` followed by ``ReLU``."""


class ConvReLU1d(_Fused):
    """``Conv1d`` followed by ``ReLU``."""


class ConvReLU3d(_Fused):
    """``Conv3d`` followed by ``ReLU``."""
