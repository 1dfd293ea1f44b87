"""Fused Conv + BatchNorm (+ ReLU) for quantization-aware training
(``lucid/nn/intrinsic/qat/modules.py:30-860``): every forward folds the BatchNorm's running
statistics into the convolution's weight, fake-quantizes the folded weight, convolves,
(ReLU,) and fake-quantizes the output.  ``convert`` bakes the folded weight into the int8
convolution of the same rank.  Forward only: training the pair is Lucid's."""

from __future__ import annotations

import numpy as np

from ... import Conv1d, Conv2d, Conv3d
from ...module import Module


class _ConvBnNd(Module):
    """Rank-generic fused Conv + BN (+ ReLU) with fold-and-fake-quant."""

    _rank = 2
    _relu = False

    def __init__(self, conv, bn, qconfig=None) -> None:
        super().__init__()
        if qconfig is None:
            raise ValueError(f"{type(self).__name__} requires a qconfig")
        want = (Conv1d, Conv2d, Conv3d)[self._rank - 1]
        if not isinstance(conv, want):
            raise TypeError(f"{type(self).__name__} needs a {want.__name__}, got {type(conv).__name__}")
        self.conv, self.bn, self.relu = conv, bn, self._relu
        self.qconfig = qconfig
        self.weight_fake_quant = qconfig.weight()
        self.activation_post_process = qconfig.activation()

    def _fold(self):
        """The BN-folded ``(weight, bias)`` as device tensors (``modules.py:52-72``): the fold of
        ``fuse_conv_bn_eval``, recomputed from the current statistics."""
        from ...utils.fusion import fuse_conv_bn_eval
        folded = fuse_conv_bn_eval(self.conv, self.bn)
        return folded.weight.to("hip"), folded.bias.to("hip")

    def forward(self, x):
        from ... import functional as F
        from ... import relu
        weight, bias = self._fold()
        w_q = self.weight_fake_quant(weight)
        conv = self.conv
        if conv.padding_mode != "zeros" or conv._padding_str == "same":
            raise NotImplementedError(f"{type(self).__name__}: zero padding with numbers (or 'valid') only")
        fn = (F.conv1d_f32, F.conv2d_f32, F.conv3d_f32)[self._rank - 1]
        y = fn(x, w_q, bias, conv.stride, conv.padding, conv.dilation, conv.groups)
        if self.relu:
            y = relu(y)
        return self.activation_post_process(y)


class ConvBn1d(_ConvBnNd):
    _rank = 1


class ConvBn2d(_ConvBnNd):
    _rank = 2


class ConvBn3d(_ConvBnNd):
    _rank = 3


class ConvBnReLU1d(_ConvBnNd):
    _rank, _relu = 1, True


class ConvBnReLU2d(_ConvBnNd):
    _rank, _relu = 2, True


class ConvBnReLU3d(_ConvBnNd):
    _rank, _relu = 3, True


def convbn_to_quantized(mod):
    """Bake a fused Conv + BN (+ ReLU) into the quantized convolution of its rank
    (``modules.py:796-857``): observe and quantize the folded weight with the module's weight
    FakeQuantize, keep the folded bias, take the output grid from its activation FakeQuantize."""
    from ... import quantized as nnq
    from ....quantization._functional import quantize
    weight, bias = mod._fold()
    wfq = mod.weight_fake_quant
    wfq(weight)
    w_scale, w_zp = wfq.calculate_qparams()
    codes = quantize(weight, w_scale, w_zp, wfq.qdtype, ch_axis=wfq.ch_axis)
    conv = mod.conv
    plain = (nnq.Conv1d, nnq.Conv2d, nnq.Conv3d)[mod._rank - 1]
    fused = (nnq.ConvReLU1d, nnq.ConvReLU2d, nnq.ConvReLU3d)[mod._rank - 1]
    pad = conv._padding_str if conv._padding_str is not None else conv.padding
    q = (fused if mod.relu else plain)(conv.in_channels, conv.out_channels, conv.kernel_size, conv.stride, pad,
                                       conv.dilation, conv.groups, bias=True)
    n = conv.out_channels
    if wfq.ch_axis is None:  # per-tensor weight qparams: one entry per output channel, as from_float keeps them
        from .... import _tensor as T_
        w_scale = T_.tensor(np.full(n, w_scale.item(), np.float32), device="hip")
        w_zp = T_.tensor(np.full(n, w_zp.item(), np.float32), device="hip")
    q.register_buffer("weight_int8", codes)
    q.register_buffer("weight_scale", w_scale.to("hip"))
    q.register_buffer("weight_zero_point", w_zp.to("hip"))
    q._state_loaded("weight_int8")
    q._state_loaded("weight_zero_point")
    q.weight_ch_axis = wfq.ch_axis if wfq.ch_axis is not None else 0
    q.register_buffer("bias", bias)
    a_scale, a_zp = mod.activation_post_process.calculate_qparams()
    q.register_buffer("scale", a_scale.to("hip"))
    q.register_buffer("zero_point", a_zp.to("hip"))
    q._state_loaded("zero_point")
    q.out_qdtype = mod.activation_post_process.qdtype
    return q


__all__ = ["ConvBn1d", "ConvBn2d", "ConvBn3d", "ConvBnReLU1d", "ConvBnReLU2d", "ConvBnReLU3d", "convbn_to_quantized"]
