"""Dynamic-quantized ``Linear`` on the hip int8 GEMM.

Mirrors ``lucid/nn/quantized/dynamic/linear.py:64-124``: buffers
``weight_int8`` / ``weight_scale`` / ``weight_zero_point`` / ``bias``,
attribute ``act_qdtype = quint8``, ``from_float(mod, dtype=qint8)``.  Per
forward: global min / max of the input -> affine qparams -> activation codes
-> int8 GEMM -> float32 output (not requantized).  All four steps are device
kernels; the activation zero point is read by the GEMM from device memory, so
the forward never waits for the host.
"""

from __future__ import annotations

import numpy as np

from .... import _C, _ops
from .... import _tensor as T
from ...._tensor import Tensor
from ....quantization._functional import minmax, quantize
from ....quantization._qparams import calculate_qparams
from ....quantization._qscheme import QDtype, per_channel_symmetric, per_tensor_affine, qint8, quint8
from ...module import Module
from .._utils import forget_weight_zero_points, storage_offset, weight_zero_points


# The one-launch kernel keeps 16 rows of activation codes (16 K bytes) plus 1 KiB of scratch in
# the 96 KiB of LDS it may use: wider layers take the two-launch route, whatever the batch.
SMALL_LINEAR_MAX_K = 6080


def fused_pair(first, relu_between: bool, second, x):
    """``second(relu(first(x)))`` (or without the ReLU) for two dynamic ``Linear`` layers on a small
    activation as ONE launch (``lq_dynamic_mlp2_small_f32``: the last block of layer 1 to finish
    reduces the hidden activation's min / max and runs layer 2), or ``None`` when the shapes or
    operands do not qualify.  Same bits as calling the modules one after the other."""
    if not (isinstance(first, Linear) and isinstance(second, Linear) and isinstance(x, Tensor)):
        return None
    if x.device != "hip" or x.dtype != T.float32 or x._grid is not None or x._range is not None:
        return None
    K1, N1, N2 = first.in_features, first.out_features, second.out_features
    if x.ndim < 1 or x.shape[-1] != K1 or second.in_features != N1:
        return None
    M = x.numel // K1
    if not (0 < M <= 64 and K1 % 16 == 0 and 16 <= K1 <= 1024 and M * K1 <= 65536 and N1 % 16 == 0
            and 16 <= N1 <= 256 and 0 < N2 <= 64):
        return None
    if first.act_qdtype is not second.act_qdtype:
        return None
    # (the buffers straight from the registries: this path is bound by what a forward costs the host)
    b1, b2 = first._buffers, second._buffers
    bias1, bias2 = b1.get("bias"), b2.get("bias")
    for lin, bias in ((first, bias1), (second, bias2)):
        if weight_zero_points(lin) is not None or (bias is not None and bias.dtype != T.float32):
            return None
        if lin._wsum is None:
            lin._wsum = _ops.rowsum_i8(lin.weight_int8)
    qd = first.act_qdtype
    y = Tensor.empty((*x.shape[:-1], N2), T.float32, "hip")
    _C.call("lq_dynamic_mlp2_small_f32", x.data_ptr, M, K1, b1["weight_int8"].data_ptr, N1, b1["weight_scale"].data_ptr,
            first._wsum.data_ptr, None if bias1 is None else bias1.data_ptr, int(relu_between),
            b2["weight_int8"].data_ptr, N2, b2["weight_scale"].data_ptr, second._wsum.data_ptr,
            None if bias2 is None else bias2.data_ptr, 0, 0, qd.quant_min, qd.quant_max, int(qd.signed),
            1e-8, storage_offset(qd), y.data_ptr, None)
    return y


class Linear(Module):
    def __init__(self, in_features: int, out_features: int, bias: bool = True) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.weight_ch_axis = 0
        self.act_qdtype: QDtype = quint8
        self.register_buffer("weight_int8", T.tensor(
            np.zeros((out_features, in_features), np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(out_features, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(
            np.zeros(out_features, np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_features, np.float32), device="hip")
                             if bias else None)
        self._wsum = None

    def _state_loaded(self, name: str) -> None:
        if name == "weight_int8":
            self._wsum = None
        if name == "weight_zero_point":
            forget_weight_zero_points(self)

    def forward(self, x: Tensor, residual: Tensor | None = None, activation: str | None = None,
                track_range: bool = False) -> Tensor:
        """Beyond Lucid's signature, all inside the GEMM epilogue: ``residual`` is added to
        the output (``x_res + linear(x)`` in one kernel); ``activation="gelu"`` applies the
        exact-erf GELU to it (``gelu(linear(x))``); ``track_range`` keeps the min / max of
        what is written, for the next dynamic-quantized layer."""
        if activation not in (None, "gelu"):
            raise ValueError(f"dynamic.Linear: unknown fused activation {activation!r}")
        if not isinstance(x, Tensor) or x.device != "hip":
            raise _C.DeviceMismatch("dynamic.Linear: input must be a tensor on the 'hip' device")
        if x.dtype != T.float32:
            raise _C.DtypeMismatch(f"dynamic.Linear expects float32 input, got {x.dtype}")
        K, N = self.in_features, self.out_features
        if x.shape[-1] != K:
            raise _C.ShapeMismatch(f"expected last dim {K}, got {x.shape}")
        M = x.numel // K
        qd = self.act_qdtype
        off = storage_offset(qd)
        if (x._range is None and residual is None and activation is None and not track_range and 0 < M <= 64
                and K % 16 == 0 and K <= SMALL_LINEAR_MAX_K and M * K <= 65536 and weight_zero_points(self) is None
                and (self.bias is None or self.bias.dtype == T.float32)):
            # a small activation: min / max, qparams, codes, GEMM and bias in one launch (same bits)
            if self._wsum is None:
                self._wsum = _ops.rowsum_i8(self.weight_int8)
            y = Tensor.empty((M, N), T.float32, "hip")
            _C.call("lq_dynamic_linear_small_f32", x.data_ptr, M, K, self.weight_int8.data_ptr, N,
                    self.weight_scale.data_ptr, self._wsum.data_ptr, None if self.bias is None else self.bias.data_ptr,
                    0, 0, qd.quant_min, qd.quant_max, int(qd.signed), 1e-8, off, y.data_ptr, None)
            return y.reshape(*x.shape[:-1], N)
        xq = Tensor.empty((M, K), T.int8, "hip")
        small = x._range is None and x.numel <= (1 << 18)
        if small:
            # min / max, qparams and codes of a small activation in one launch (same bits)
            x_scale = Tensor.empty((), T.float32, "hip")
            x_zp = Tensor.empty((), T.float32, "hip")
            _C.call("lq_quantize_tensor_dynamic_i8", x.data_ptr if x.numel else None, x.numel, 0, qd.quant_min,
                    qd.quant_max, int(qd.signed), 1e-8, off, x_scale.data_ptr, x_zp.data_ptr, None, None,
                    xq.data_ptr if x.numel else None, None)
        elif x._range is not None:
            # the kernel that wrote x kept its min / max: qparams straight from them
            x_scale = Tensor.empty((), T.float32, "hip")
            x_zp = Tensor.empty((), T.float32, "hip")
            _C.call("lq_calc_qparams_from_range", x._range.data_ptr, 0, qd.quant_min, qd.quant_max,
                    int(qd.signed), 1e-8, x_scale.data_ptr, x_zp.data_ptr, None, None, None)
        else:
            mn, mx = minmax(x)
            x_scale, x_zp = calculate_qparams(mn, mx, per_tensor_affine, qd)
        if not small:
            _C.call("lq_quantize", x.data_ptr, xq.data_ptr, _C.I8, off, 1, 1, x.numel,
                    x_scale.data_ptr, x_zp.data_ptr, 0, qd.quant_min, qd.quant_max, None)
        return self.forward_quantized(xq, x_scale, x_zp, x.shape[:-1], residual, activation, track_range)

    def forward_quantized(self, xq: Tensor, x_scale: Tensor, x_zp: Tensor, lead_shape, residual: Tensor | None = None,
                          activation: str | None = None, track_range: bool = False) -> Tensor:
        """The layer on an activation that is already quantized with this layer's activation
        grid (``act_qdtype``, per-tensor affine, device-side ``x_scale`` / ``x_zp``): what
        ``forward`` does after its own quantization, for a producer that writes codes directly
        (``functional.layer_norm_dynamic_quantize``)."""
        N = self.out_features
        off = storage_offset(self.act_qdtype)
        if self._wsum is None:
            self._wsum = _ops.rowsum_i8(self.weight_int8)
        rng = None
        w_zp = weight_zero_points(self)
        if track_range and w_zp is not None:
            raise NotImplementedError("dynamic.Linear: track_range (an extension of this backend) is "
                                      "not available with affine weights")
        if track_range:
            from ...functional import _new_range
            rng = _new_range()
        y = _ops.qlinear_i8(xq, self.weight_int8, a_zp=off, a_zp_dev=x_zp, a_scale=x_scale,
                            w_scale=self.weight_scale, wsum=self._wsum, bias=self.bias,
                            out_mode=_ops.OUT_F32, residual=residual, gelu=activation == "gelu",
                            range_buf=rng, w_zp=w_zp)
        y = y.reshape(*lead_shape, N)
        y._range = rng
        return y

    @classmethod
    def from_float(cls, mod, dtype: QDtype = qint8) -> "Linear":
        """Quantize a float ``Linear``'s weight, no calibration
        (``dynamic/linear.py:101-120``)."""
        from ....quantization.observer import PerChannelMinMaxObserver

        qmod = cls(mod.in_features, mod.out_features, bias=mod.bias is not None)
        weight = mod.weight.to("hip")
        obs = PerChannelMinMaxObserver(ch_axis=0, qscheme=per_channel_symmetric, qdtype=dtype)
        obs(weight)
        scale, zero_point = obs.calculate_qparams()
        if dtype.storage != "int8":
            raise NotImplementedError(f"dynamic.Linear weights must use int8 storage, got {dtype!r}")
        qmod.register_buffer("weight_int8", quantize(weight, scale, zero_point, dtype, ch_axis=0))
        qmod.register_buffer("weight_scale", scale)
        qmod.register_buffer("weight_zero_point", zero_point)
        if mod.bias is not None:
            qmod.register_buffer("bias", mod.bias.to("hip"))
        return qmod

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, dynamic=True"
