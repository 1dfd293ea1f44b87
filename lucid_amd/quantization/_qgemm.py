"""Group-wise weight-only int4 / int8 (``lucid/quantization/_qgemm.py:24-320``):
``quantize`` packs a float weight, ``dequantize`` inverts it, ``quantized_matmul``
contracts a float activation against the packed weight.  Lucid runs these on MLX
(Metal); here they are HIP kernels with the same signatures, defaults and shapes.
The packed tensor is int32-tagged (Lucid has no uint32 dtype either,
``QuantizedMatmul.cpp:53-63``).
"""

from __future__ import annotations

from .. import _C
from .. import _tensor as T
from .._tensor import Tensor


def is_available() -> bool:
    """True when the HIP library and a device are present (``_qgemm.py:24-66``)."""
    return _C.is_available()


def _check(name: str, *ts: Tensor) -> None:
    for t in ts:
        if not isinstance(t, Tensor) or t.device != "hip":
            raise _C.DeviceMismatch(f"{name}: operands must be tensors on the 'hip' device")


def quantize(w: Tensor, group_size: int = 64, bits: int = 8) -> tuple[Tensor, Tensor, Tensor]:
    """``(packed_weight, scales, biases)`` of a float32 ``(out, in)`` weight."""
    _check("quantize", w)
    if w.dtype != T.float32 or w.ndim != 2:
        raise _C.DtypeMismatch(f"quantize expects a 2-d float32 weight, got {w.dtype} {w.shape}")
    N, K = w.shape
    packed = Tensor.empty((N, K * bits // 32), T.int32, "hip")
    scales = Tensor.empty((N, K // group_size), T.float32, "hip")
    biases = Tensor.empty((N, K // group_size), T.float32, "hip")
    _C.call("lq_wq_quantize", w.data_ptr, N, K, int(group_size), int(bits), packed.data_ptr,
            scales.data_ptr, biases.data_ptr, None)
    return packed, scales, biases


def dequantize(wq: Tensor, scales: Tensor, biases: Tensor, group_size: int = 64, bits: int = 8) -> Tensor:
    """Float32 ``(out, in)`` weight ``c * s + beta``."""
    _check("dequantize", wq, scales, biases)
    N = wq.shape[0]
    K = wq.shape[1] * 32 // bits
    out = Tensor.empty((N, K), T.float32, "hip")
    _C.call("lq_wq_dequantize", wq.data_ptr, scales.data_ptr, biases.data_ptr, N, K, int(group_size),
            int(bits), out.data_ptr, None)
    return out


def quantized_matmul(x: Tensor, wq: Tensor, scales: Tensor, biases: Tensor, transpose: bool = True,
                     group_size: int = 64, bits: int = 8) -> Tensor:
    """``x @ w_hat.T`` (``transpose=True``, the Linear layout); float32 in and out."""
    _check("quantized_matmul", x, wq, scales, biases)
    if not transpose:
        raise NotImplementedError("quantized_matmul on hip: only transpose=True (x @ w_hat.T) is built")
    if x.dtype != T.float32:
        raise _C.DtypeMismatch(f"quantized_matmul expects a float32 activation, got {x.dtype}")
    N = wq.shape[0]
    K = wq.shape[1] * 32 // bits
    if x.shape[-1] != K:
        raise _C.ShapeMismatch(f"quantized_matmul: activation {x.shape} against a packed ({N}, {K}) weight")
    M = x.numel // K
    out = Tensor.empty((*x.shape[:-1], N), T.float32, "hip")
    _C.call("lq_wq_matmul", x.data_ptr, wq.data_ptr, scales.data_ptr, biases.data_ptr, M, N, K,
            int(group_size), int(bits), out.data_ptr, None)
    return out
