"""QAT ``Conv2d`` / ``ConvReLU2d`` (``lucid/nn/qat/conv.py``): fake-quantize the kernel, run the
float convolution, (ReLU,) fake-quantize the output.  Zero padding with symmetric amounts."""

from __future__ import annotations

from .. import Conv2d as _FloatConv2d


class Conv2d(_FloatConv2d):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, padding_mode="zeros", qconfig=None) -> None:
        super().__init__(in_channels, out_channels, kernel_size, stride, padding, dilation, groups, bias, padding_mode)
        if qconfig is None:
            raise ValueError("nn.qat.Conv2d needs a qconfig (prepare_qat provides it)")
        self.qconfig = qconfig
        self.weight_fake_quant = qconfig.weight()
        self.activation_post_process = qconfig.activation()

    def _conv(self, x):
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        kept = self._buffers["weight"]
        try:  # the float layer's forward on the fake-quantized kernel
            self._buffers["weight"] = self.weight_fake_quant(w)
            return _FloatConv2d.forward(self, x)
        finally:
            self._buffers["weight"] = kept

    def forward(self, x):
        return self.activation_post_process(self._conv(x))

    @classmethod
    def from_float(cls, mod) -> "Conv2d":
        pad = mod._padding_str if mod._padding_str is not None else mod.padding
        qat = cls(mod.in_channels, mod.out_channels, mod.kernel_size, mod.stride, pad, mod.dilation, mod.groups,
                  bias=mod.bias is not None, padding_mode=mod.padding_mode, qconfig=mod.qconfig)
        qat.register_buffer("weight", mod.weight.to("hip"))
        if mod.bias is not None:
            qat.register_buffer("bias", mod.bias.to("hip"))
        return qat


class ConvReLU2d(Conv2d):
    def forward(self, x):
        from .. import relu
        return self.activation_post_process(relu(self._conv(x)))

    @classmethod
    def from_float(cls, mod) -> "ConvReLU2d":
        inner = mod[0]
        inner.qconfig = mod.qconfig
        return super().from_float(inner)
