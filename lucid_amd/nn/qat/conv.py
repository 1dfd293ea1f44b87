"""QAT convolutions (``lucid/nn/qat/conv.py``): ``Conv1d / Conv2d / Conv3d`` and their
``ConvReLU`` forms.  A forward fake-quantizes the kernel, runs the float convolution on the
device, (ReLU,) and fake-quantizes the output.  Zero padding with symmetric amounts."""

from __future__ import annotations

from .. import Conv1d as _FloatConv1d
from .. import Conv2d as _FloatConv2d
from .. import Conv3d as _FloatConv3d


class _QatConvMixin:
    """The QAT behaviour shared by the three ranks; the float parent supplies the convolution."""

    _float_cls = None

    def _init_qat(self, qconfig) -> None:
        if qconfig is None:
            raise ValueError(f"nn.qat.{type(self).__name__} needs a qconfig (prepare_qat provides it)")
        self.qconfig = qconfig
        self.weight_fake_quant = qconfig.weight()
        self.activation_post_process = qconfig.activation()

    def _conv(self, x):
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        kept = self._buffers["weight"]
        try:  # the float layer's forward on the fake-quantized kernel
            self._buffers["weight"] = self.weight_fake_quant(w)
            return self._float_cls.forward(self, x)
        finally:
            self._buffers["weight"] = kept

    def forward(self, x):
        return self.activation_post_process(self._conv(x))

    @classmethod
    def from_float(cls, mod):
        pad = mod._padding_str if mod._padding_str is not None else mod.padding
        qat = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, pad, mod.dilation, mod.groups,
                  bias=mod.bias is not None, padding_mode=mod.padding_mode, qconfig=mod.qconfig)
        qat.register_buffer("weight", mod.weight.to("hip"))
        if mod.bias is not None:
            qat.register_buffer("bias", mod.bias.to("hip"))
        return qat


class _QatConvReLUMixin:
    def forward(self, x):
        from .. import relu
        return self.activation_post_process(relu(self._conv(x)))

    @classmethod
    def from_float(cls, mod):
        if not hasattr(mod, "__getitem__"):
            return super().from_float(mod)
        inner = mod[0]
        inner.qconfig = mod.qconfig
        return super().from_float(inner)


def _make(float_cls, name):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode="zeros", qconfig=None) -> None:
        float_cls.__init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias,
                           padding_mode)
        self._init_qat(qconfig)
    return type(name, (_QatConvMixin, float_cls), {"__init__": __init__, "_float_cls": float_cls,
                                                   "__doc__": f"QAT ``{name}``: fake-quantized kernel and output."})


Conv1d = _make(_FloatConv1d, "Conv1d")
Conv2d = _make(_FloatConv2d, "Conv2d")
Conv3d = _make(_FloatConv3d, "Conv3d")
for _c in (Conv1d, Conv2d, Conv3d):
    _c.__module__ = __name__


class ConvReLU1d(_QatConvReLUMixin, Conv1d):
    """QAT ``Conv1d`` + ``ReLU`` (``qat/conv.py:476``)."""


class ConvReLU2d(_QatConvReLUMixin, Conv2d):
    """QAT ``Conv2d`` + ``ReLU`` (``qat/conv.py:586``)."""


class ConvReLU3d(_QatConvReLUMixin, Conv3d):
    """QAT ``Conv3d`` + ``ReLU`` (``qat/conv.py:697``)."""
