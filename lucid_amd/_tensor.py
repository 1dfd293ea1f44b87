"""Minimal tensor handle for the ``hip`` device.

Lucid's ``Tensor`` wraps a C++ ``TensorImpl`` whose ``Storage`` is a variant of
CPU / GPU / shared storage (``lucid/_C/core/Storage.h:334``).  This package
adds a third storage kind - a HIP device allocation - and only what the
quantized-inference path needs around it: shape, dtype, upload / download.

A ``"cpu"`` tensor here is a host container (numpy array) used to stage data
in and out; every compute entry point requires ``device == "hip"`` and raises
``DeviceMismatch`` otherwise, so nothing ever computes on the host.
"""

from __future__ import annotations

import ctypes as C
import math
import weakref
from dataclasses import dataclass

import numpy as np

from . import _C


# ---------------------------------------------------------------- dtypes
@dataclass(frozen=True)
class dtype:
    """Element type; ``code`` is Lucid's ``Dtype`` enum value (``core/Dtype.h``)."""

    name: str
    code: int
    itemsize: int
    np: object

    def __repr__(self) -> str:
        return f"lucid.{self.name}"


bool_ = dtype("bool", _C.BOOL, 1, np.bool_)
int8 = dtype("int8", _C.I8, 1, np.int8)
int16 = dtype("int16", _C.I16, 2, np.int16)
int32 = dtype("int32", _C.I32, 4, np.int32)
int64 = dtype("int64", _C.I64, 8, np.int64)
float16 = dtype("float16", _C.F16, 2, np.float16)
float32 = dtype("float32", _C.F32, 4, np.float32)
float64 = dtype("float64", _C.F64, 8, np.float64)

_ALL = (bool_, int8, int16, int32, int64, float16, float32, float64)
_BY_NP = {np.dtype(d.np): d for d in _ALL}
_BY_NAME = {d.name: d for d in _ALL}


def as_dtype(d) -> dtype:
    if isinstance(d, dtype):
        return d
    if isinstance(d, str):
        return _BY_NAME[d]
    return _BY_NP[np.dtype(d)]


# ---------------------------------------------------------------- devices
# lucid/_device.py:21-22 knows "cpu" and "metal"; this backend adds "hip".
_KNOWN_DEVICES = ("cpu", "hip")


def _norm_device(device) -> str:
    d = str(device).split(":")[0]
    if d not in _KNOWN_DEVICES:
        raise ValueError(f"unknown device {device!r}; expected one of {_KNOWN_DEVICES}")
    return d


class Grid:
    """Quantization-grid tag of an activation.

    Lucid carries a quantized activation as a *float* tensor that happens to
    lie on its grid (``lucid/nn/quantized/linear.py:207-215``).  Here the same
    value is carried as its int8 codes plus ``(scale, zero_point)``; the float
    view ``(code - Z) * S`` is produced by ``lq_dequantize`` only when somebody
    asks for it.  ``offset`` is what was added to the code when storing it
    (-128 for ``quint8``, so the codes are valid signed MFMA operands).
    ``layout`` is "plain" (same element order as the float view) or "nhwc"
    (codes of an NCHW / NCDHW float tensor kept channel-last for the conv kernels).
    """

    __slots__ = ("codes", "scale", "zero_point", "qdtype", "offset", "zp_host", "layout")

    def __init__(self, codes, scale, zero_point, qdtype, offset, zp_host=None, layout="plain"):
        self.codes, self.scale, self.zero_point = codes, scale, zero_point
        self.qdtype, self.offset, self.zp_host, self.layout = qdtype, offset, zp_host, layout


class DeviceBuffer:
    """Owns one ``lq_alloc`` allocation; freed when the last reference dies."""

    __slots__ = ("ptr", "nbytes", "_fin", "__weakref__")

    def __init__(self, nbytes: int) -> None:
        _C.init()
        p = C.c_void_p()
        _C.call("lq_alloc", C.byref(p), int(nbytes))
        self.ptr = p.value
        self.nbytes = int(nbytes)
        self._fin = weakref.finalize(self, _free, self.ptr)


def _free(ptr) -> None:
    try:
        _C.load().lq_free(ptr)
    except Exception:  # interpreter shutdown
        pass


class Tensor:
    """Contiguous row-major tensor on ``"hip"`` (device memory) or ``"cpu"``
    (host staging)."""

    __slots__ = ("shape", "dtype", "device", "_buf", "_host", "_offset", "_grid", "_range", "__weakref__")

    def __init__(self, shape, dt, device, buf=None, host=None, offset=0) -> None:
        self.shape = tuple(int(s) for s in shape)
        self.dtype = as_dtype(dt)
        self.device = _norm_device(device)
        self._buf = buf
        self._host = host
        self._offset = int(offset)
        self._grid = None  # set by ops whose result lies on a quantization grid
        # device min / max keys kept by the kernel that wrote this tensor
        # (``lq_range_keys_init``), read by a dynamic quantizer downstream
        self._range = None

    # -- construction
    @staticmethod
    def empty(shape, dt=float32, device="hip") -> "Tensor":
        dt = as_dtype(dt)
        shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        n = math.prod(shape)
        if _norm_device(device) == "cpu":
            return Tensor(shape, dt, "cpu", host=np.empty(shape, dt.np))
        return Tensor(shape, dt, "hip", buf=DeviceBuffer(n * dt.itemsize))

    @staticmethod
    def from_numpy(a, device="hip") -> "Tensor":
        a = np.asarray(a)
        if not a.flags.c_contiguous:  # (np.ascontiguousarray would also turn 0-d into 1-d)
            a = np.ascontiguousarray(a)
        dt = as_dtype(a.dtype)
        if _norm_device(device) == "cpu":
            return Tensor(a.shape, dt, "cpu", host=a)
        t = Tensor.empty(a.shape, dt, "hip")
        _C.call("lq_h2d", t.data_ptr, a.ctypes.data, a.nbytes, None)
        return t

    # -- properties
    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def numel(self) -> int:
        return math.prod(self.shape)

    @property
    def nbytes(self) -> int:
        return self.numel * self.dtype.itemsize

    @property
    def data_ptr(self) -> int:
        if self.device != "hip":
            raise _C.DeviceMismatch("data_ptr: tensor is not on the hip device")
        if self._buf is None:
            self._materialize()
        return self._buf.ptr + self._offset

    @staticmethod
    def on_grid(shape, grid: "Grid") -> "Tensor":
        """A float32 tensor whose value is given by codes on a grid; the float
        storage is created on first use."""
        t = Tensor(shape, float32, "hip", buf=None)
        t._grid = grid
        return t

    def _materialize(self) -> None:
        g = self._grid
        if g is None:
            raise _C.LucidError("tensor has no storage")
        n = self.numel
        buf = DeviceBuffer(n * 4)
        if g.layout == "nhwc" and len(self.shape) in (4, 5):
            # (B, C, H, W) or (B, C, D, H, W): the kernel only needs the number of positions per image
            B, Cc = self.shape[:2]
            H, W = int(np.prod(self.shape[2:-1], dtype=np.int64)), self.shape[-1]
            _C.call("lq_dequantize_nhwc_to_nchw", g.codes.data_ptr, g.offset, buf.ptr, B, Cc, H, W,
                    g.scale.data_ptr, g.zero_point.data_ptr, None)
        else:
            _C.call("lq_dequantize", g.codes.data_ptr, _C.I8, g.offset, buf.ptr, 1, 1, n,
                    g.scale.data_ptr, g.zero_point.data_ptr, 0, None)
        self._buf = buf

    @property
    def is_hip(self) -> bool:
        return self.device == "hip"

    def size(self, dim=None):
        return self.shape if dim is None else self.shape[dim]

    def __len__(self) -> int:
        return self.shape[0]

    def __repr__(self) -> str:
        return f"Tensor(shape={self.shape}, dtype={self.dtype.name}, device='{self.device}')"

    # -- movement
    def numpy(self) -> np.ndarray:
        if self.device == "cpu":
            return self._host
        out = np.empty(self.shape, self.dtype.np)
        if out.nbytes:
            _C.call("lq_d2h", out.ctypes.data, self.data_ptr, out.nbytes, None)
        return out

    def to(self, target) -> "Tensor":
        """``.to("hip")`` / ``.to("cpu")`` (``lucid/_tensor/_to.py:125-199``), or ``.to(dtype)``:
        the engine's ``astype`` on the device, numpy's on the host."""
        if isinstance(target, dtype):
            if target == self.dtype:
                return self
            if self.device == "cpu":
                return Tensor(self.shape, target, "cpu", host=self._host.astype(target.np))
            from ._engine_ops import astype
            return astype(self, target)
        dev = _norm_device(target)
        if dev == self.device:
            return self
        if dev == "hip":
            t = Tensor.from_numpy(self._host, "hip")
        else:
            t = Tensor.from_numpy(self.numpy(), "cpu")
        return t

    def copy_from(self, a) -> "Tensor":
        """Overwrite this tensor's storage with a host array of the same shape
        and dtype (the way to feed a new batch to a captured graph)."""
        a = np.asarray(a, dtype=self.dtype.np)
        if not a.flags.c_contiguous:
            a = np.ascontiguousarray(a)
        if a.shape != self.shape:
            raise _C.ShapeMismatch(f"copy_from: {a.shape} into {self.shape}")
        if self.device == "cpu":
            self._host[...] = a
        elif a.nbytes:
            _C.call("lq_h2d", self.data_ptr, a.ctypes.data, a.nbytes, None)
        return self

    def cpu(self) -> "Tensor":
        return self.to("cpu")

    def item(self):
        if self.numel != 1:
            raise ValueError("item() needs a one-element tensor")
        return self.numpy().reshape(()).item()

    def tolist(self):
        return self.numpy().tolist()

    def reshape(self, *shape) -> "Tensor":
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        shape = list(shape)
        if -1 in shape:
            known = math.prod(s for s in shape if s != -1)
            shape[shape.index(-1)] = self.numel // max(known, 1)
        if math.prod(shape) != self.numel:
            raise _C.ShapeMismatch(f"cannot reshape {self.shape} to {tuple(shape)}")
        if self.device == "cpu":
            return Tensor(shape, self.dtype, "cpu", host=self._host.reshape(shape))
        g = self._grid
        if g is not None and g.layout == "plain":
            # keep the grid tag: the codes are reshaped the same way
            out = Tensor(shape, self.dtype, "hip", buf=self._buf, offset=self._offset)
            out._grid = Grid(g.codes.reshape(shape), g.scale, g.zero_point, g.qdtype, g.offset,
                             g.zp_host, "plain")
            return out
        if self._buf is None:
            self._materialize()
        return Tensor(shape, self.dtype, "hip", buf=self._buf, offset=self._offset)

    def narrow_rows(self, n: int) -> "Tensor":
        """The first ``n`` entries along axis 0 as a view of the same storage (a prefix of a
        contiguous tensor is contiguous)."""
        if self.device != "hip" or self._grid is not None:
            raise NotImplementedError("narrow_rows: plain device tensors only")
        if not 0 <= n <= self.shape[0]:
            raise _C.ShapeMismatch(f"narrow_rows: {n} rows of {self.shape[0]}")
        return Tensor((n, *self.shape[1:]), self.dtype, "hip", buf=self._buf, offset=self._offset)

    def row_range(self, lo: int, hi: int) -> "Tensor":
        """Entries ``[lo, hi)`` along axis 0 as a view of the same storage."""
        if self.device != "hip" or self._grid is not None:
            raise NotImplementedError("row_range: plain device tensors only")
        if not 0 <= lo <= hi <= self.shape[0]:
            raise _C.ShapeMismatch(f"row_range: [{lo}, {hi}) of {self.shape[0]}")
        if self._buf is None:
            self._materialize()
        row_bytes = self.nbytes // self.shape[0] if self.shape[0] else 0
        return Tensor((hi - lo, *self.shape[1:]), self.dtype, "hip", buf=self._buf,
                      offset=self._offset + lo * row_bytes)

    def detach(self) -> "Tensor":
        return self

    # -- arithmetic: one engine call per operator, on float32 device tensors
    def __add__(self, other):
        from . import _engine_ops as E
        return E.add(self, other)

    __radd__ = __add__

    def __sub__(self, other):
        from . import _engine_ops as E
        return E.sub(self, other)

    def __rsub__(self, other):
        from . import _engine_ops as E
        return E.sub(other, self)

    def __mul__(self, other):
        from . import _engine_ops as E
        return E.mul(self, other)

    __rmul__ = __mul__

    def __truediv__(self, other):
        from . import _engine_ops as E
        return E.div(self, other)

    def __rtruediv__(self, other):
        from . import _engine_ops as E
        return E.div(other, self)

    def min(self, dim=None, keepdim: bool = False) -> "Tensor":
        from . import _engine_ops as E
        return E.amin(self, dim, keepdim)

    def max(self, dim=None, keepdim: bool = False) -> "Tensor":
        from . import _engine_ops as E
        return E.amax(self, dim, keepdim)

    def round(self) -> "Tensor":
        from . import _engine_ops as E
        return E.round(self)

    def clip(self, min_v, max_v) -> "Tensor":
        from . import _engine_ops as E
        return E.clip(self, min_v, max_v)

    def clone(self) -> "Tensor":
        if self.device == "cpu":
            return Tensor(self.shape, self.dtype, "cpu", host=self._host.copy())
        out = Tensor.empty(self.shape, self.dtype, "hip")
        if self.nbytes:
            _C.call("lq_d2d", out.data_ptr, self.data_ptr, self.nbytes, None)
        return out

    def __deepcopy__(self, memo) -> "Tensor":
        # a device allocation has exactly one owner: copy the bytes, not the handle
        return self.clone()


def tensor(data, dtype=None, device="cpu") -> Tensor:
    """``lucid.tensor``: Python floats become float32, ints int64 - unless
    ``dtype`` says otherwise."""
    a = np.asarray(data)
    if dtype is not None:
        a = a.astype(as_dtype(dtype).np)
    elif a.dtype == np.float64:
        a = a.astype(np.float32)
    return Tensor.from_numpy(a, device)


def is_floating_point(t: Tensor) -> bool:
    return t.dtype in (float16, float32, float64)


def synchronize() -> None:
    _C.call("lq_sync", None)
