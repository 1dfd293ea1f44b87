"""``QuantizedLinearMLX`` (``lucid/nn/quantized/mlx_linear.py:21-200``): a Linear whose
weight is group-wise int4 / int8 packed and decoded inside the matmul.  The name is
Lucid's; on this backend the kernels are HIP.  Buffers as in Lucid:
``packed_weight`` int32 ``(out, in*bits/32)``, ``scales`` / ``biases`` float32
``(out, in/group_size)``, ``bias`` float32 ``(out,)`` or None; attributes ``bits``,
``group_size``, ``relu``.
"""

from __future__ import annotations

import numpy as np

from ... import _C
from ... import _tensor as T
from ..._tensor import Tensor
from ...quantization import _qgemm
from ..module import Module


class QuantizedLinearMLX(Module):
    def __init__(self, in_features: int, out_features: int, bias: bool = True, bits: int = 8,
                 group_size: int = 64, relu: bool = False) -> None:
        super().__init__()
        if bits not in (4, 8):
            raise ValueError(f"bits must be 4 or 8, got {bits}")
        if in_features % group_size:
            raise ValueError(f"group_size {group_size} must divide in_features {in_features}")
        self.in_features, self.out_features = in_features, out_features
        self.bits, self.group_size, self.relu = bits, group_size, relu
        self.register_buffer("packed_weight", T.tensor(
            np.zeros((out_features, in_features * bits // 32), np.int32), device="hip"))
        g = in_features // group_size
        self.register_buffer("scales", T.tensor(np.zeros((out_features, g), np.float32), device="hip"))
        self.register_buffer("biases", T.tensor(np.zeros((out_features, g), np.float32), device="hip"))
        self.register_buffer("bias", T.tensor(np.zeros(out_features, np.float32), device="hip") if bias else None)

    def forward(self, x: Tensor) -> Tensor:
        if not isinstance(x, Tensor) or x.device != "hip":
            raise _C.DeviceMismatch("QuantizedLinearMLX: input must be a tensor on the 'hip' device")
        y = _qgemm.quantized_matmul(x, self.packed_weight, self.scales, self.biases, transpose=True,
                                    group_size=self.group_size, bits=self.bits)
        if self.bias is not None or self.relu:
            M = y.numel // self.out_features
            _C.call("lq_bias_act_f32", y.data_ptr, self.bias.data_ptr if self.bias is not None else None,
                    M, self.out_features, int(self.relu), None)
        return y

    @classmethod
    def from_float(cls, mod, bits: int = 8, group_size: int = 64, relu: bool = False) -> "QuantizedLinearMLX":
        """Pack a float ``Linear``'s weight (``mlx_linear.py`` ``from_float``)."""
        q = cls(mod.in_features, mod.out_features, bias=mod.bias is not None, bits=bits,
                group_size=group_size, relu=relu)
        packed, scales, biases = _qgemm.quantize(mod.weight.to("hip"), group_size, bits)
        q.register_buffer("packed_weight", packed)
        q.register_buffer("scales", scales)
        q.register_buffer("biases", biases)
        if mod.bias is not None:
            q.register_buffer("bias", mod.bias.to("hip"))
        return q

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, bits={self.bits}, "
                f"group_size={self.group_size}")
