"""QAT ``Linear`` / ``LinearReLU`` (``lucid/nn/qat/linear.py:157-178,281-293``): fake-quantize
the weight, run the float linear, (ReLU,) fake-quantize the output."""

from __future__ import annotations

import numpy as np

from ... import _tensor as T
from ..module import Module


class Linear(Module):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, qconfig=None) -> None:
        super().__init__()
        if qconfig is None:
            raise ValueError("nn.qat.Linear needs a qconfig (prepare_qat provides it)")
        self.in_features, self.out_features = in_features, out_features
        self.qconfig = qconfig
        self.register_buffer("weight", T.tensor(np.zeros((out_features, in_features), np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_features, np.float32), device="hip") if bias else None)
        self.weight_fake_quant = qconfig.weight()
        self.activation_post_process = qconfig.activation()

    def _linear(self, x):
        from ..functional import linear_f32
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        b = self.bias
        if b is not None and b.device != "hip":
            b = b.to("hip")
        return linear_f32(x, self.weight_fake_quant(w), b)

    def forward(self, x):
        return self.activation_post_process(self._linear(x))

    @classmethod
    def from_float(cls, mod) -> "Linear":
        """A QAT layer that adopts the float layer's weight and bias (``linear.py:163-178``)."""
        qat = cls(mod.in_features, mod.out_features, bias=mod.bias is not None, qconfig=mod.qconfig)
        qat.register_buffer("weight", mod.weight.to("hip"))
        if mod.bias is not None:
            qat.register_buffer("bias", mod.bias.to("hip"))
        return qat

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}"


class LinearReLU(Linear):
    def forward(self, x):
        from .. import relu
        return self.activation_post_process(relu(self._linear(x)))

    @classmethod
    def from_float(cls, mod) -> "LinearReLU":
        """From a fused float ``nni.LinearReLU`` (its inner linear, ``linear.py:287-293``)."""
        inner = mod[0]
        inner.qconfig = mod.qconfig
        return super().from_float(inner)
