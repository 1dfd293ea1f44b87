"""The engine primitives Lucid's quantization composites are written in, on ``"hip"``
tensors: one library call per ``IBackend`` call (``lucid/_C/backend/IBackend.h:370-374,
433-434,474,689-692,1232,2121``).

With these, the composite of ``lucid/quantization/_functional.py:180`` runs as written,

    codes = clip(round(x / s) + z, qdtype.quant_min, qdtype.quant_max).to(int8)

through ``Tensor.__truediv__`` / ``__add__`` / ``.to(dtype)`` and the functions below:
call for call what Lucid's engine does (broadcast materialisation included), and bit for
bit what the fused ``lq_quantize`` gives in one pass.  The modules never take this route;
it exists for unmodified composite code and as the fused kernels' specification.
"""

from __future__ import annotations

import ctypes as C

import numpy as np

from . import _C
from . import _tensor as T
from ._tensor import Tensor


def _hip_f32(t, what: str) -> Tensor:
    if not isinstance(t, Tensor) or t.device != "hip":
        raise _C.DeviceMismatch(f"{what}: expected a tensor on the 'hip' device")
    if t.dtype != T.float32:
        raise _C.DtypeMismatch(f"{what} expects float32, got {t.dtype}")
    if t._grid is not None:
        t._materialize()
    return t


def broadcast_to(t: Tensor, shape) -> Tensor:
    """Materialise ``t`` at ``shape`` (``kernel/BinaryKernel.h:591-606``).  ``t``'s extents
    other than 1 must form one run of neighbouring axes that match ``shape`` there - a
    scalar, or a per-channel vector after ``_reshape_for_channel``."""
    shape = tuple(int(s) for s in shape)
    if tuple(t.shape) == shape:
        return t
    src = (1,) * (len(shape) - t.ndim) + tuple(t.shape)
    if len(src) != len(shape) or any(a != b and a != 1 for a, b in zip(src, shape)):
        raise _C.ShapeMismatch(f"cannot broadcast {t.shape} to {shape}")
    live = [i for i, a in enumerate(src) if a != 1]
    if live and live != list(range(live[0], live[-1] + 1)):
        raise NotImplementedError(f"broadcast of {t.shape} to {shape}: the kept axes must be neighbours")
    lo, hi = (live[0], live[-1] + 1) if live else (0, 0)
    outer = int(np.prod(shape[:lo], dtype=np.int64))
    c = int(np.prod(shape[lo:hi], dtype=np.int64))
    inner = int(np.prod(shape[hi:], dtype=np.int64))
    out = Tensor.empty(shape, T.float32, "hip")
    _C.call("lq_broadcast_f32", t.data_ptr, out.data_ptr, outer, c, inner, None)
    return out


def _operand(v, what: str) -> Tensor:
    """A Python number becomes a one-element device tensor, as the engine fills a scalar
    operand; a host tensor is moved to the device."""
    if isinstance(v, Tensor):
        return _hip_f32(v if v.device == "hip" else v.to("hip"), what)
    if isinstance(v, (int, float, np.floating, np.integer)):
        return T.tensor(np.float32(v), device="hip")
    raise TypeError(f"{what}: unsupported operand {type(v).__name__}")


def _binary(name: str, a, b) -> Tensor:
    a, b = _operand(a, name), _operand(b, name)
    shape = tuple(np.broadcast_shapes(tuple(a.shape), tuple(b.shape)))
    a, b = broadcast_to(a, shape), broadcast_to(b, shape)
    out = Tensor.empty(shape, T.float32, "hip")
    _C.call(f"lq_{name}_f32", a.data_ptr, b.data_ptr, out.data_ptr, out.numel, None)
    return out


def add(a, b) -> Tensor:
    return _binary("add", a, b)


def sub(a, b) -> Tensor:
    return _binary("sub", a, b)


def mul(a, b) -> Tensor:
    return _binary("mul", a, b)


def div(a, b) -> Tensor:
    return _binary("div", a, b)


def maximum(a, b) -> Tensor:
    return _binary("maximum", a, b)


def minimum(a, b) -> Tensor:
    return _binary("minimum", a, b)


def round(x: Tensor) -> Tensor:  # noqa: A001 - Lucid's name
    """``lucid.round``: ties to even."""
    x = _hip_f32(x, "round")
    out = Tensor.empty(x.shape, T.float32, "hip")
    _C.call("lq_round_f32", x.data_ptr, out.data_ptr, x.numel, None)
    return out


def clip(x: Tensor, min_v: float, max_v: float) -> Tensor:
    """``lucid.clip``: bounds cast to float32, NaN passes through."""
    x = _hip_f32(x, "clip")
    out = Tensor.empty(x.shape, T.float32, "hip")
    _C.call("lq_clip_f32", x.data_ptr, out.data_ptr, x.numel, float(min_v), float(max_v), None)
    return out


_ASTYPE = ("int8", "int16", "int32", "float16", "float32")


def astype(x: Tensor, dt) -> Tensor:
    """``Tensor.to(dtype)`` on the device (``IBackend::astype``)."""
    dt = T.as_dtype(dt)
    if not isinstance(x, Tensor) or x.device != "hip":
        raise _C.DeviceMismatch("astype: expected a tensor on the 'hip' device")
    if x._grid is not None:
        x._materialize()
    if x.dtype.name not in _ASTYPE or dt.name not in _ASTYPE:
        raise NotImplementedError(f"astype {x.dtype} -> {dt}: the hip backend converts between {_ASTYPE}")
    out = Tensor.empty(x.shape, dt, "hip")
    _C.call("lq_astype", x.data_ptr, x.dtype.code, out.data_ptr, dt.code, x.numel, None)
    return out


def _reduce(x: Tensor, dim, keepdim: bool) -> tuple[Tensor, Tensor]:
    x = _hip_f32(x, "min / max")
    nd = x.ndim
    if dim is None:
        axes = list(range(nd))
    else:
        dims = dim if isinstance(dim, (tuple, list)) else (dim,)
        if any(not -nd <= d < nd for d in dims):
            raise ValueError(f"min / max: dim {dim} out of range for a {nd}-d tensor")
        axes = sorted({d % nd for d in dims})
    kept = [s for i, s in enumerate(x.shape) if i not in axes]
    full = [1 if i in axes else s for i, s in enumerate(x.shape)]
    mn = Tensor.empty(tuple(kept), T.float32, "hip")
    mx = Tensor.empty(tuple(kept), T.float32, "hip")
    shape = (C.c_int64 * max(nd, 1))(*x.shape)
    ax = (C.c_int * max(len(axes), 1))(*axes)
    _C.call("lq_reduce_minmax", x.data_ptr, shape, nd, ax, len(axes), mn.data_ptr, mx.data_ptr, None)
    if keepdim:
        mn, mx = mn.reshape(full), mx.reshape(full)
    return mn, mx


def amin(x: Tensor, dim=None, keepdim: bool = False) -> Tensor:
    """``x.min()`` / ``lucid.amin(x, dim)`` (``IBackend::reduce_min``), NaN-propagating."""
    return _reduce(x, dim, keepdim)[0]


def amax(x: Tensor, dim=None, keepdim: bool = False) -> Tensor:
    return _reduce(x, dim, keepdim)[1]


def batch_norm_eval(x: Tensor, running_mean: Tensor, running_var: Tensor, weight, bias, eps: float) -> Tensor:
    """``F.batch_norm(..., training=False)`` (``lucid/nn/functional/normalization.py:104-109``)
    on a ``(N, C, *)`` float32 device tensor."""
    x = _hip_f32(x, "batch_norm")
    if x.ndim < 2 or x.ndim > 5:
        raise ValueError(f"batch_norm: expected 2-5D input, got ndim={x.ndim}")
    Cn = x.shape[1]
    dev = lambda t: None if t is None else (t if t.device == "hip" else t.to("hip"))
    rm, rv, w, b = dev(running_mean), dev(running_var), dev(weight), dev(bias)
    for t, name in ((rm, "running_mean"), (rv, "running_var"), (w, "weight"), (b, "bias")):
        if t is not None and (t.numel != Cn or t.dtype != T.float32):
            raise _C.ShapeMismatch(f"batch_norm: {name} must hold {Cn} float32 values, got {t.shape} {t.dtype}")
    spatial = int(np.prod(x.shape[2:], dtype=np.int64))
    out = Tensor.empty(x.shape, T.float32, "hip")
    _C.call("lq_batchnorm_eval_f32", x.data_ptr, out.data_ptr, x.shape[0], Cn, spatial, rm.data_ptr, rv.data_ptr,
            None if w is None else w.data_ptr, None if b is None else b.data_ptr, float(eps), None)
    return out
