"""The slice of ``lucid.nn`` that the quantized-inference path touches.

Float ``Conv2d`` and friends here are parameter holders that ``from_float`` /
``quantize_dynamic`` / ``convert`` read; their float forward is Lucid's CPU /
Metal business and is not part of this backend (calling it raises).  ``Linear``,
``ReLU`` and the pointwise activations do compute in float32 on the device, so that
a prepared MLP can be calibrated where it will run.
"""

from __future__ import annotations

import numpy as np

from .. import _C
from .. import _tensor as T
from .._tensor import Tensor
from .module import Module


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


class Identity(Module):
    def forward(self, x):
        return x


def _fused_dynamic_pair(mods, i, x):
    """``(result, next index)`` when the modules at ``i`` are Linear [, ReLU], Linear from
    ``nn.quantized.dynamic`` on an activation small enough for the one-launch kernel, else ``None``
    (no hooks on the modules: a hook has to see each module's own output).

    Not while a graph is being captured.  The one launch (15.7 us of kernel for 784-256-10 at
    batch 64: layer 2 waits for the last block of layer 1 through device-scope memory) saves the
    host a launch, which is what a Python-driven forward is bound by; the two separate layers are
    8 + 6 us of kernels, and a replayed graph, which pays its launch cost once whichever it holds,
    is shorter with those: 25 against 31 us.  Same bits either way."""
    from .quantized.dynamic import linear as _dyn
    from .. import graph as _graph

    if _graph.is_capturing():
        return None
    first = mods[i]
    if type(first) is not _dyn.Linear or i + 1 >= len(mods):
        return None
    relu = type(mods[i + 1]) is ReLU
    j = i + 2 if relu else i + 1
    if j >= len(mods) or type(mods[j]) is not _dyn.Linear:
        return None
    for m in mods[i:j + 1]:
        d = m.__dict__  # (not getattr: a name a module lacks costs an exception inside Module.__getattr__)
        if d.get("_forward_hooks") or d.get("_forward_pre_hooks"):
            return None
    y = _dyn.fused_pair(first, relu, mods[j], x)
    return None if y is None else (y, j + 1)


class Sequential(Module):
    def __init__(self, *mods) -> None:
        super().__init__()
        for i, m in enumerate(mods):
            self._modules[str(i)] = m

    def __getitem__(self, i):
        return list(self._modules.values())[i]

    def __len__(self):
        return len(self._modules)

    def forward(self, x):
        mods = list(self._modules.values())
        i = 0
        while i < len(mods):
            # two small dynamic-quantized Linears in a row, with or without a ReLU between: one launch
            skip = _fused_dynamic_pair(mods, i, x)
            if skip is not None:
                x, i = skip
                continue
            x = mods[i](x)
            i += 1
        return x


class Linear(Module):
    """Float Linear as a parameter holder (``weight`` (out,in), ``bias`` (out,))."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True) -> None:
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        bound = 1.0 / np.sqrt(in_features)
        rng = np.random.default_rng(in_features * 7919 + out_features)
        self.register_buffer("weight", T.tensor(
            rng.uniform(-bound, bound, (out_features, in_features)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_features).astype(np.float32)) if bias else None)

    def forward(self, x):
        """``x @ weight.T + bias`` in float32 on the device - what a calibration pass
        through a prepared model needs (observers are forward hooks)."""
        if not isinstance(x, Tensor) or x.device != "hip":
            raise NotImplementedError(
                "float nn.Linear.forward runs on the 'hip' device only; the CPU float path is Lucid's")
        from .functional import linear_f32
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        b = self.bias
        if b is not None and b.device != "hip":
            b = b.to("hip")
        return linear_f32(x, w, b)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}"


class Conv2d(Module):
    """Float Conv2d as a parameter holder (``weight`` OIHW, ``bias`` (O,))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros") -> None:
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = _pair(kernel_size), _pair(stride)
        self.dilation, self.groups = _pair(dilation), groups
        self._padding_str = padding if isinstance(padding, str) else None
        self.padding = (0, 0) if isinstance(padding, str) else _pair(padding)
        self.padding_mode = padding_mode
        fan_in = in_channels // groups * self.kernel_size[0] * self.kernel_size[1]
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + out_channels)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (out_channels, in_channels // groups, *self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        """Float32 convolution on the device (im2col + GEMM): what a calibration pass through a
        prepared model needs.  Zero padding with symmetric amounts; inference is the quantized
        module's business."""
        if not isinstance(x, Tensor) or x.device != "hip":
            raise NotImplementedError(
                "float nn.Conv2d.forward runs on the 'hip' device only; the CPU float path is Lucid's")
        if self.padding_mode != "zeros":
            raise NotImplementedError(f"float nn.Conv2d.forward: padding_mode {self.padding_mode!r} is not built")
        pad = self.padding
        if self._padding_str == "same":
            from .quantized.conv import _same_pad_pair
            ph = _same_pad_pair(x.shape[2], self.kernel_size[0], self.stride[0], self.dilation[0])
            pw = _same_pad_pair(x.shape[3], self.kernel_size[1], self.stride[1], self.dilation[1])
            if ph[0] != ph[1] or pw[0] != pw[1]:
                raise NotImplementedError("float nn.Conv2d.forward: asymmetric 'same' padding is not built")
            pad = (ph[0], pw[0])
        from .functional import conv2d_f32
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        b = self.bias
        if b is not None and b.device != "hip":
            b = b.to("hip")
        return conv2d_f32(x, w, b, self.stride, pad, self.dilation, self.groups)


class Conv1d(Module):
    """Float Conv1d as a parameter holder (``weight`` (O, I/groups, K), ``bias`` (O,))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros") -> None:
        super().__init__()
        one = lambda v: int(v[0]) if isinstance(v, (tuple, list)) else int(v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = one(kernel_size), one(stride)
        self.dilation, self.groups = one(dilation), groups
        self._padding_str = padding if isinstance(padding, str) else None
        self.padding = 0 if isinstance(padding, str) else one(padding)
        self.padding_mode = padding_mode
        fan_in = in_channels // groups * self.kernel_size
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + out_channels + 1)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (out_channels, in_channels // groups, self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        """Float32 convolution on the device: the 2-d kernel on a one-row image."""
        if not isinstance(x, Tensor) or x.device != "hip":
            raise NotImplementedError(
                "float nn.Conv1d.forward runs on the 'hip' device only; the CPU float path is Lucid's")
        if self.padding_mode != "zeros" or self._padding_str == "same":
            raise NotImplementedError("float nn.Conv1d.forward: zero padding with a number (or 'valid') only")
        if x.ndim != 3 or x.shape[1] != self.in_channels:
            raise _C.ShapeMismatch(f"Conv1d: expected (B, {self.in_channels}, L), got {x.shape}")
        from .functional import conv1d_f32
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        b = self.bias
        if b is not None and b.device != "hip":
            b = b.to("hip")
        return conv1d_f32(x, w, b, self.stride, self.padding, self.dilation, self.groups)


class Conv3d(Module):
    """Float Conv3d as a parameter holder (``weight`` (O, I/groups, KD, KH, KW), ``bias`` (O,))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode="zeros") -> None:
        super().__init__()
        three = lambda v: (int(v),) * 3 if isinstance(v, int) else tuple(int(e) for e in v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = three(kernel_size), three(stride)
        self.dilation, self.groups = three(dilation), groups
        self._padding_str = padding if isinstance(padding, str) else None
        self.padding = (0, 0, 0) if isinstance(padding, str) else three(padding)
        self.padding_mode = padding_mode
        fan_in = in_channels // groups * int(np.prod(self.kernel_size))
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + out_channels + 3)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (out_channels, in_channels // groups, *self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        """Float32 convolution on the device (depth taps summed over 2-d convolutions of depth
        slices): calibration and QAT forwards of volumetric models.  Zero padding, symmetric."""
        if not isinstance(x, Tensor) or x.device != "hip":
            raise NotImplementedError(
                "float nn.Conv3d.forward runs on the 'hip' device only; the CPU float path is Lucid's")
        if self.padding_mode != "zeros":
            raise NotImplementedError(f"float nn.Conv3d.forward: padding_mode {self.padding_mode!r} is not built")
        pad = self.padding
        if self._padding_str == "same":
            from .quantized.conv import _same_pad_pair
            pairs = [_same_pad_pair(n, k, s, d)
                     for n, k, s, d in zip(x.shape[2:], self.kernel_size, self.stride, self.dilation)]
            if any(lo != hi for lo, hi in pairs):
                raise NotImplementedError("float nn.Conv3d.forward: asymmetric 'same' padding is not built")
            pad = tuple(lo for lo, _ in pairs)
        from .functional import conv3d_f32
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        b = self.bias
        if b is not None and b.device != "hip":
            b = b.to("hip")
        return conv3d_f32(x, w, b, self.stride, pad, self.dilation, self.groups)


class _BatchNorm(Module):
    """Float BatchNorm: the parameter / statistics holder that ``fuse_modules`` folds into the
    preceding convolution, and the eval-mode forward on the device
    (``lucid/nn/modules/normalization.py`` ``_BatchNormBase``; ``F.batch_norm`` with
    ``training=False``).  Training-mode statistics are Lucid's."""

    _ndim = (4,)

    def __init__(self, num_features: int, eps: float = 1e-5, momentum: float = 0.1, affine: bool = True) -> None:
        super().__init__()
        self.num_features, self.eps, self.momentum, self.affine = num_features, eps, momentum, affine
        self.register_buffer("weight", T.tensor(np.ones(num_features, np.float32)) if affine else None)
        self.register_buffer("bias", T.tensor(np.zeros(num_features, np.float32)) if affine else None)
        self.register_buffer("running_mean", T.tensor(np.zeros(num_features, np.float32)))
        self.register_buffer("running_var", T.tensor(np.ones(num_features, np.float32)))

    def forward(self, x):
        if getattr(self, "training", False):
            raise NotImplementedError(
                f"float nn.{type(self).__name__}.forward in training mode (batch statistics) is Lucid's; "
                "call .eval() - the hip backend runs the frozen-statistics forward")
        if not isinstance(x, Tensor) or x.device != "hip":
            raise NotImplementedError(
                f"float nn.{type(self).__name__}.forward runs on the 'hip' device only; the CPU float path is Lucid's")
        if x.ndim not in self._ndim or x.shape[1] != self.num_features:
            raise _C.ShapeMismatch(f"{type(self).__name__}: expected {self._ndim}-d input with "
                                   f"{self.num_features} channels, got {x.shape}")
        from .._engine_ops import batch_norm_eval
        return batch_norm_eval(x, self.running_mean, self.running_var, self.weight if self.affine else None,
                               self.bias if self.affine else None, self.eps)

    def extra_repr(self) -> str:
        return f"{self.num_features}, eps={self.eps}, affine={self.affine}"


class BatchNorm1d(_BatchNorm):
    _ndim = (2, 3)


class BatchNorm2d(_BatchNorm):
    _ndim = (4,)


class BatchNorm3d(_BatchNorm):
    _ndim = (5,)


def relu(x: Tensor) -> Tensor:
    """``F.relu``.  On a grid-carried activation with a non-negative grid the
    codes are clamped at the zero point instead of touching floats."""
    if not isinstance(x, Tensor) or x.device != "hip":
        raise _C.DeviceMismatch("relu: expected a tensor on the 'hip' device")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"relu expects float32, got {x.dtype}")
    out = Tensor.empty(x.shape, T.float32, "hip")
    _C.call("lq_relu_f32", x.data_ptr, out.data_ptr, x.numel, None)
    return out


class ReLU(Module):
    def forward(self, x):
        return relu(x)


class MaxPool2d(Module):
    """``F.max_pool2d`` on a grid-carried NCHW activation: pooling the codes
    equals pooling the values (quantization is monotone), so the result stays on
    the input's grid."""

    def __init__(self, kernel_size, stride=None, padding=0) -> None:
        super().__init__()
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride if stride is not None else kernel_size)
        self.padding = _pair(padding)

    def forward(self, x: Tensor) -> Tensor:
        g = x._grid if isinstance(x, Tensor) else None
        if g is None or g.layout != "nhwc":
            raise NotImplementedError("MaxPool2d: only grid-carried NCHW activations are supported")
        B, H, W, Cc = g.codes.shape
        (kh, kw), (sh, sw), (ph, pw) = self.kernel_size, self.stride, self.padding
        OH, OW = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
        out = Tensor.empty((B, OH, OW, Cc), T.int8, "hip")
        _C.call("lq_maxpool2d_nhwc_i8", g.codes.data_ptr, out.data_ptr, B, H, W, Cc, kh, kw, sh, sw,
                ph, pw, None)
        return Tensor.on_grid((B, Cc, OH, OW), T.Grid(out, g.scale, g.zero_point, g.qdtype, g.offset,
                                                      g.zp_host, "nhwc"))


class AdaptiveAvgPool2d(Module):
    """``F.adaptive_avg_pool2d(x, 1)``: the mean of the float-carried values,
    which leaves the grid - the result is an ordinary float tensor (B, C, 1, 1)."""

    def __init__(self, output_size=1) -> None:
        super().__init__()
        if _pair(output_size) != (1, 1):
            raise NotImplementedError("AdaptiveAvgPool2d: only global pooling (output_size=1)")

    def forward(self, x: Tensor) -> Tensor:
        g = x._grid if isinstance(x, Tensor) else None
        if g is None or g.layout != "nhwc":
            raise NotImplementedError(
                "AdaptiveAvgPool2d: only grid-carried NCHW activations are supported")
        B, H, W, Cc = g.codes.shape
        out = Tensor.empty((B, Cc, 1, 1), T.float32, "hip")
        _C.call("lq_global_avgpool_nhwc_i8", g.codes.data_ptr, g.offset, B, H, W, Cc,
                g.scale.data_ptr, g.zero_point.data_ptr, out.data_ptr, None)
        return out


class Flatten(Module):
    def __init__(self, start_dim: int = 1) -> None:
        super().__init__()
        self.start_dim = start_dim

    def forward(self, x):
        lead = x.shape[: self.start_dim]
        return x.reshape(*lead, -1)


from . import intrinsic, quantized, utils  # noqa: E402  (sub-packages need the classes above)


class LayerNorm(Module):
    """``nn.LayerNorm`` over the last axis, float32, one HIP kernel."""

    def __init__(self, normalized_shape: int, eps: float = 1e-5, track_range: bool = False) -> None:
        super().__init__()
        self.normalized_shape, self.eps = int(normalized_shape), float(eps)
        self.track_range = track_range  # keep min / max of the output for a dynamic quantizer
        self.register_buffer("weight", T.tensor(np.ones(normalized_shape, np.float32)))
        self.register_buffer("bias", T.tensor(np.zeros(normalized_shape, np.float32)))

    def forward(self, x):
        from . import functional as F

        return F.layer_norm(x, self.normalized_shape, self.weight, self.bias, self.eps, self.track_range)


class GELU(Module):
    def forward(self, x):
        from . import functional as F

        return F.gelu(x)


class Embedding(Module):
    """Float Embedding as a parameter holder (``weight`` (num_embeddings, embedding_dim))."""

    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int | None = None) -> None:
        super().__init__()
        self.num_embeddings, self.embedding_dim, self.padding_idx = num_embeddings, embedding_dim, padding_idx
        rng = np.random.default_rng(num_embeddings * 7919 + embedding_dim)
        w = rng.standard_normal((num_embeddings, embedding_dim)).astype(np.float32)
        if padding_idx is not None:
            w[padding_idx] = 0.0
        self.register_buffer("weight", T.tensor(w))

    def forward(self, x):
        raise NotImplementedError(
            "float nn.Embedding.forward is not part of the hip quantized-inference backend; "
            "convert the model first")

    def extra_repr(self) -> str:
        return f"{self.num_embeddings}, {self.embedding_dim}"


class EmbeddingBag(Embedding):
    """Float EmbeddingBag as a parameter holder; ``mode`` in ``sum`` / ``mean`` / ``max``."""

    def __init__(self, num_embeddings: int, embedding_dim: int, mode: str = "mean",
                 padding_idx: int | None = None) -> None:
        super().__init__(num_embeddings, embedding_dim, padding_idx)
        if mode not in ("sum", "mean", "max"):
            raise ValueError(f"EmbeddingBag: mode must be one of ['max', 'mean', 'sum'], got {mode!r}")
        self.mode = mode


class _FloatActivation(Module):
    """Float activation evaluated by the same kernel as its quantized form, without the
    output grid."""

    _kind = -1

    def _alpha(self) -> float:
        return 0.0

    def forward(self, x: Tensor) -> Tensor:
        from .quantized.activation import apply_activation
        return apply_activation(self._kind, self._alpha(), x, None)


class Sigmoid(_FloatActivation):
    _kind = 0


class Hardswish(_FloatActivation):
    _kind = 1


class Hardsigmoid(_FloatActivation):
    _kind = 2


class Tanh(_FloatActivation):
    _kind = 3


class ELU(_FloatActivation):
    _kind = 4

    def __init__(self, alpha: float = 1.0) -> None:
        super().__init__()
        self.alpha = float(alpha)

    def _alpha(self) -> float:
        return self.alpha


class LeakyReLU(_FloatActivation):
    _kind = 5

    def __init__(self, negative_slope: float = 0.01) -> None:
        super().__init__()
        self.negative_slope = float(negative_slope)

    def _alpha(self) -> float:
        return self.negative_slope


class ConvTranspose2d(Module):
    """Float ConvTranspose2d as a parameter holder (``weight`` (in, out/groups, kh, kw))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1) -> None:
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = _pair(kernel_size), _pair(stride)
        self.padding = padding if isinstance(padding, str) else _pair(padding)
        self.output_padding, self.dilation, self.groups = _pair(output_padding), _pair(dilation), groups
        fan_in = out_channels // groups * self.kernel_size[0] * self.kernel_size[1]
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + in_channels)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (in_channels, out_channels // groups, *self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        raise NotImplementedError(
            "float nn.ConvTranspose2d.forward is not part of the hip quantized-inference backend; "
            "quantize the model (convert) first")


class ConvTranspose1d(Module):
    """Float ConvTranspose1d as a parameter holder (``weight`` (in, out/groups, k))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1) -> None:
        super().__init__()
        one = lambda v: int(v[0]) if isinstance(v, (tuple, list)) else int(v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = one(kernel_size), one(stride)
        self.padding = padding if isinstance(padding, str) else one(padding)
        self.output_padding, self.dilation, self.groups = one(output_padding), one(dilation), groups
        fan_in = out_channels // groups * self.kernel_size
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + in_channels + 1)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (in_channels, out_channels // groups, self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        raise NotImplementedError(
            "float nn.ConvTranspose1d.forward is not part of the hip quantized-inference backend; "
            "quantize the model (convert) first")


class ConvTranspose3d(Module):
    """Float ConvTranspose3d as a parameter holder (``weight`` (in, out/groups, kd, kh, kw))."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, output_padding=0,
                 groups=1, bias=True, dilation=1) -> None:
        super().__init__()
        three = lambda v: (int(v),) * 3 if isinstance(v, int) else tuple(int(e) for e in v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = three(kernel_size), three(stride)
        self.padding = padding if isinstance(padding, str) else three(padding)
        self.output_padding, self.dilation, self.groups = three(output_padding), three(dilation), groups
        fan_in = out_channels // groups * int(np.prod(self.kernel_size))
        bound = 1.0 / np.sqrt(fan_in)
        rng = np.random.default_rng(fan_in * 7919 + in_channels + 3)
        self.register_buffer("weight", T.tensor(rng.uniform(
            -bound, bound, (in_channels, out_channels // groups, *self.kernel_size)).astype(np.float32)))
        self.register_buffer("bias", T.tensor(
            rng.uniform(-bound, bound, out_channels).astype(np.float32)) if bias else None)

    def forward(self, x):
        raise NotImplementedError(
            "float nn.ConvTranspose3d.forward is not part of the hip quantized-inference backend; "
            "quantize the model (convert) first")


class LSTM(Module):
    """Float LSTM as a parameter holder: ``weight_ih_l{k}`` (4H, in), ``weight_hh_l{k}``
    (4H, H or proj_size), ``bias_ih_l{k}``, ``bias_hh_l{k}``, ``weight_hr_l{k}`` (proj_size, H)
    when ``proj_size > 0`` (and ``..._reverse`` when bidirectional), gate order i, f, g, o."""

    def __init__(self, input_size: int, hidden_size: int, num_layers: int = 1, bias: bool = True,
                 batch_first: bool = False, dropout: float = 0.0, bidirectional: bool = False,
                 proj_size: int = 0) -> None:
        super().__init__()
        if proj_size < 0 or (proj_size > 0 and proj_size >= hidden_size):
            raise ValueError(f"proj_size ({proj_size}) must be in [0, hidden_size = {hidden_size})")
        self.input_size, self.hidden_size, self.num_layers = input_size, hidden_size, num_layers
        self.bias, self.batch_first, self.dropout = bias, batch_first, dropout
        self.bidirectional, self.proj_size = bidirectional, proj_size
        rec = proj_size if proj_size > 0 else hidden_size  # what re-enters the recurrence
        bound = 1.0 / np.sqrt(hidden_size)
        rng = np.random.default_rng(input_size * 7919 + hidden_size * 31 + num_layers)
        dirs = 2 if bidirectional else 1
        for k in range(num_layers):
            fan = input_size if k == 0 else rec * dirs
            for suffix in ("", "_reverse")[:dirs]:
                u = lambda *shape: T.tensor(rng.uniform(-bound, bound, shape).astype(np.float32))
                self.register_buffer(f"weight_ih_l{k}{suffix}", u(4 * hidden_size, fan))
                self.register_buffer(f"weight_hh_l{k}{suffix}", u(4 * hidden_size, rec))
                if bias:
                    self.register_buffer(f"bias_ih_l{k}{suffix}", u(4 * hidden_size))
                    self.register_buffer(f"bias_hh_l{k}{suffix}", u(4 * hidden_size))
                if proj_size > 0:  # W_hr: (proj_size, hidden_size), rnn.py:541-549
                    self.register_buffer(f"weight_hr_l{k}{suffix}", u(proj_size, hidden_size))

    def named_parameters(self):
        return list(self.named_buffers())

    def forward(self, x, hx=None):
        raise NotImplementedError(
            "float nn.LSTM.forward is not part of the hip quantized-inference backend; "
            "quantize the model (quantize_dynamic) first")
