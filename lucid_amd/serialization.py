"""Checkpoints of quantized modules in Lucid's two wire formats.

``save`` / ``load`` write and read the ``.lucid`` container of
``lucid/serialization/__init__.py``: a pickle stream of
``{"_lucid_format": 2, "obj": obj}`` in which every tensor is a persistent id
``("tensor_v3", shape, dtype_name, device, raw_bytes)`` - the engine's
``to_bytes`` / ``from_bytes`` contract (``lucid/_C/bindings/bind_tensor.cpp:152-160``):
contiguous row-major little-endian bytes.  ``load`` only ever uses the restricted
unpickler (Lucid's ``weights_only=True`` whitelist), so a file cannot run code.

``save_safetensors`` / ``load_safetensors`` write and read the SafeTensors layout
(8-byte little-endian header length, JSON header, raw data) with Lucid's
convention for 0-d tensors: stored as shape ``(1,)`` and listed in the
``__lucid_scalar_keys__`` metadata entry (``serialization/__init__.py:588-597``).

Device memory never appears in a file: ``hip`` tensors are written as ``"cpu"``
(Lucid knows ``"cpu"`` and ``"metal"`` only), so checkpoints made here load in
Lucid and the other way round; ``Module.load_state_dict`` puts each loaded
tensor on the device of the buffer it replaces.  Buffer names and dtypes of the
quantized modules are Lucid's (``weight_int8`` int8, ``weight_scale`` /
``weight_zero_point`` float32 ``(N,)``, ``scale`` / ``zero_point`` float32 0-d,
``bias`` float32; ``lucid/nn/quantized/linear.py:183-193``).
"""

from __future__ import annotations

import io
import json
import pickle
import struct
from collections import OrderedDict

import numpy as np

from ._tensor import Tensor, as_dtype

_SAFE_CLASSES = frozenset({
    "builtins.dict", "builtins.list", "builtins.tuple", "builtins.int", "builtins.float",
    "builtins.str", "builtins.bool", "builtins.bytes", "builtins.NoneType", "collections.OrderedDict",
})


class _Pickler(pickle.Pickler):
    def persistent_id(self, obj):
        if isinstance(obj, Tensor):
            return ("tensor_v3", list(obj.shape), obj.dtype.name, "cpu", np.asarray(obj.numpy()).tobytes())
        return None


class _SafeUnpickler(pickle.Unpickler):
    def __init__(self, f, device: str) -> None:
        super().__init__(f)
        self._device = device

    def find_class(self, module, name):
        full = f"{module}.{name}"
        if full in _SAFE_CLASSES:
            return super().find_class(module, name)
        raise pickle.UnpicklingError(f"refusing to deserialize {full!r}: only plain containers and "
                                     "tensors are allowed in a checkpoint")

    def persistent_load(self, pid):
        if isinstance(pid, tuple) and pid and pid[0] in ("tensor_v3", "tensor"):
            shape, dtype_name, raw = pid[1], pid[2], pid[4]
            dt = as_dtype(dtype_name)
            a = np.frombuffer(raw, dtype=dt.np).reshape(tuple(shape)).copy()
            return Tensor.from_numpy(a, self._device)
        raise pickle.UnpicklingError(f"unknown persistent id: {pid!r}")


def save(obj, f, *, pickle_protocol: int = 4) -> None:
    """``lucid.save``: write ``obj`` (normally a ``state_dict``) as a ``.lucid`` file."""
    container = {"_lucid_format": 2, "obj": obj}
    meta = getattr(obj, "_metadata", None)
    if meta is not None:
        container["_state_dict_metadata"] = meta
    buf = io.BytesIO()
    _Pickler(buf, protocol=pickle_protocol).dump(container)
    if isinstance(f, (str, bytes)):
        with open(f, "wb") as fp:
            fp.write(buf.getvalue())
    else:
        f.write(buf.getvalue())


def load(f, *, map_location: str = "cpu"):
    """``lucid.load`` with ``weights_only=True`` semantics (always).  Tensors come
    back on ``map_location`` (``"cpu"`` or ``"hip"``)."""
    if isinstance(f, (str, bytes)):
        path = f.decode() if isinstance(f, bytes) else str(f)
        if path.endswith(".safetensors"):
            return load_safetensors(path, device=map_location)
        with open(path, "rb") as fp:
            data = fp.read()
    else:
        data = f.read()
    container = _SafeUnpickler(io.BytesIO(data), map_location).load()
    if not isinstance(container, dict) or container.get("_lucid_format") not in (1, 2):
        raise RuntimeError("File is not a valid Lucid checkpoint")
    return container["obj"]


# SafeTensors dtype tags for the dtypes this package has
_ST_TAG = {"bool": "BOOL", "int8": "I8", "int16": "I16", "int32": "I32", "int64": "I64",
           "float16": "F16", "float32": "F32", "float64": "F64"}
_ST_NAME = {v: k for k, v in _ST_TAG.items()}


def save_safetensors(state_dict, path: str, *, metadata: dict | None = None) -> None:
    """``lucid.serialization.save_safetensors``: flat dict of tensors only."""
    header, blobs, at, scalars = OrderedDict(), [], 0, []
    for name, t in state_dict.items():
        if not isinstance(t, Tensor):
            raise TypeError(f"save_safetensors: state_dict[{name!r}] is {type(t).__name__}, expected Tensor")
        a = np.asarray(t.numpy())
        if a.ndim == 0:  # SafeTensors has no 0-d tensors: store (1,) and tag the key
            a = a.reshape((1,))
            scalars.append(name)
        raw = a.tobytes()  # C-order bytes whatever the array's strides
        header[name] = {"dtype": _ST_TAG[t.dtype.name], "shape": list(a.shape), "data_offsets": [at, at + len(raw)]}
        blobs.append(raw)
        at += len(raw)
    meta = dict(metadata) if metadata else {}
    if scalars:
        meta["__lucid_scalar_keys__"] = ",".join(scalars)
    out = OrderedDict()
    if meta:
        out["__metadata__"] = {str(k): str(v) for k, v in meta.items()}
    out.update(header)
    hdr = json.dumps(out, separators=(",", ":")).encode("utf-8")
    hdr += b" " * (-len(hdr) % 8)  # data starts 8-byte aligned, as the reference writer does
    with open(path, "wb") as fp:
        fp.write(struct.pack("<Q", len(hdr)))
        fp.write(hdr)
        for raw in blobs:
            fp.write(raw)


def load_safetensors(path: str, *, device: str = "cpu") -> dict:
    """``lucid.serialization.load_safetensors``; ``device`` is ``"cpu"`` or ``"hip"``."""
    with open(path, "rb") as fp:
        (n,) = struct.unpack("<Q", fp.read(8))
        if n > 100 * 1024 * 1024:
            raise RuntimeError("safetensors header is implausibly large")
        header = json.loads(fp.read(n).decode("utf-8"))
        data = fp.read()
    meta = header.pop("__metadata__", {}) or {}
    scalars = set(meta.get("__lucid_scalar_keys__", "").split(",")) - {""}
    out = {}
    for name, ent in header.items():
        lo, hi = ent["data_offsets"]
        dt = as_dtype(_ST_NAME[ent["dtype"]])
        a = np.frombuffer(data[lo:hi], dtype=dt.np).reshape(tuple(ent["shape"])).copy()
        if name in scalars:
            a = a.reshape(())
        out[name] = Tensor.from_numpy(a, device)
    return out
