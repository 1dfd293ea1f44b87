"""``FakeQuantize`` (``lucid/quantization/_fake_quantize.py:29-260``): an observer plus the
fake-quantize transform in one module - what ``prepare_qat`` puts on weights and activations.

Forward only.  On this backend the module serves to *evaluate* a QAT-prepared model (the
simulated-quantization forward, bit for bit the composition ``observer`` ->
``calculate_qparams`` -> ``fake_quantize`` of the hip kernels) and to ``convert`` it; the
straight-through gradient of ``_functional.py:334-448`` belongs to training, which this
backend does not do.
"""

from __future__ import annotations

import functools

from .. import _tensor as T
from ..nn.module import Module
from ._functional import fake_quantize
from .observer import MovingAverageMinMaxObserver


class FakeQuantize(Module):
    def __init__(self, observer=MovingAverageMinMaxObserver, **observer_kwargs) -> None:
        super().__init__()
        self.activation_post_process = observer(**observer_kwargs)
        self.qdtype = self.activation_post_process.qdtype
        self.qscheme = self.activation_post_process.qscheme
        self.ch_axis = self.activation_post_process.ch_axis
        import numpy as np
        self.register_buffer("scale", T.tensor(np.float32(1.0), device="hip"))
        self.register_buffer("zero_point", T.tensor(np.float32(0.0), device="hip"))
        self._observer_enabled = True
        self._fake_quant_enabled = True

    def forward(self, x):
        """Refresh the qparams (if observing), then fake-quantize (if enabled)."""
        if self._observer_enabled:
            self.activation_post_process(x)
            scale, zero_point = self.activation_post_process.calculate_qparams()
            self.register_buffer("scale", scale)
            self.register_buffer("zero_point", zero_point)
        if self._fake_quant_enabled:
            return fake_quantize(x, self.scale, self.zero_point, self.qdtype.quant_min, self.qdtype.quant_max,
                                 self.ch_axis)
        return x

    def enable_observer(self, enabled: bool = True) -> "FakeQuantize":
        self._observer_enabled = enabled
        return self

    def disable_observer(self) -> "FakeQuantize":
        return self.enable_observer(False)

    def enable_fake_quant(self, enabled: bool = True) -> "FakeQuantize":
        self._fake_quant_enabled = enabled
        return self

    def disable_fake_quant(self) -> "FakeQuantize":
        return self.enable_fake_quant(False)

    def calculate_qparams(self):
        return self.activation_post_process.calculate_qparams()

    @classmethod
    def with_args(cls, **kwargs):
        return functools.partial(cls, **kwargs)
