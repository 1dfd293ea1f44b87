"""Quantized ``Embedding`` / ``EmbeddingBag`` (``lucid/nn/quantized/sparse.py:22-336``):
an int8 table with one scale per row.  Lucid dequantizes the whole table on every
forward and then gathers; here the kernel reads only the rows that are asked for and
decodes them on the way out - the same values, without touching the rest of the table.
"""

from __future__ import annotations


import numpy as np

from ... import _C
from ... import _tensor as T
from ..._tensor import Tensor
from ...quantization._functional import quantize
from ...quantization._qscheme import per_channel_symmetric, qint8
from ..module import Module
from ._utils import quantize_weight

_MODES = {"sum": 0, "mean": 1, "max": 2}


def check_embedding_indices(x: Tensor, num_embeddings: int, op: str) -> None:
    """``lucid/nn/functional/sparse.py:17-71``: TypeError for non-integer indices,
    IndexError (same text) for an index outside the table."""
    if not isinstance(x, Tensor) or x.device != "hip":
        raise _C.DeviceMismatch(f"{op}: indices must be a tensor on the 'hip' device")
    if x.dtype not in (T.int32, T.int64):
        if T.is_floating_point(x):
            raise TypeError(f"{op}: indices must be an integer tensor, got {x.dtype}; "
                            "cast with .to(lucid.int64) first")
        raise NotImplementedError(f"{op}: indices must be int32 or int64 on the hip device, got {x.dtype}")
    if x.numel == 0:
        return
    out = Tensor.empty((2,), T.int64, "hip")
    _C.call("lq_index_minmax", x.data_ptr, int(x.dtype is T.int64), x.numel, out.data_ptr, None)
    lo, hi = (int(v) for v in out.numpy())
    if lo < 0 or hi >= num_embeddings:
        bad = lo if lo < 0 else hi
        raise IndexError(f"{op}: index {bad} is out of range for a table with {num_embeddings} entries "
                         f"(valid range [0, {num_embeddings - 1}])")


def _quantize_table(mod):
    """Per-row symmetric qint8 codes of a float table (``sparse.py:141-156``)."""
    if getattr(mod, "qconfig", None) is None:
        from ...quantization.observer import PerChannelMinMaxObserver
        obs = PerChannelMinMaxObserver(ch_axis=0, qscheme=per_channel_symmetric, qdtype=qint8)
        w = mod.weight.to("hip")
        obs(w)
        scale, zero_point = obs.calculate_qparams()
        return quantize(w, scale, zero_point, qint8, ch_axis=0), scale.to("hip"), zero_point.to("hip")
    codes, scale, zero_point, _ = quantize_weight(mod)
    return codes, scale, zero_point


class Embedding(Module):
    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int | None = None) -> None:
        super().__init__()
        self.num_embeddings, self.embedding_dim, self.padding_idx = num_embeddings, embedding_dim, padding_idx
        self.weight_ch_axis = 0
        self.register_buffer("weight_int8", T.tensor(np.zeros((num_embeddings, embedding_dim), np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(num_embeddings, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(np.zeros(num_embeddings, np.float32), device="hip"))

    def forward(self, x: Tensor) -> Tensor:
        check_embedding_indices(x, self.num_embeddings, "embedding")
        out = Tensor.empty(tuple(x.shape) + (self.embedding_dim,), T.float32, "hip")
        _C.call("lq_embedding_i8", self.weight_int8.data_ptr, self.weight_scale.data_ptr,
                self.weight_zero_point.data_ptr, self.num_embeddings, self.embedding_dim, x.data_ptr,
                int(x.dtype is T.int64), x.numel, -1 if self.padding_idx is None else int(self.padding_idx),
                out.data_ptr, None)
        return out

    @classmethod
    def from_float(cls, mod) -> "Embedding":
        q = cls(mod.num_embeddings, mod.embedding_dim, padding_idx=mod.padding_idx)
        codes, scale, zero_point = _quantize_table(mod)
        q.register_buffer("weight_int8", codes)
        q.register_buffer("weight_scale", scale)
        q.register_buffer("weight_zero_point", zero_point)
        return q

    def extra_repr(self) -> str:
        return f"num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim}"


class EmbeddingBag(Module):
    def __init__(self, num_embeddings: int, embedding_dim: int, mode: str = "mean",
                 padding_idx: int | None = None) -> None:
        super().__init__()
        self.num_embeddings, self.embedding_dim = num_embeddings, embedding_dim
        self.mode, self.padding_idx = mode, padding_idx
        self.weight_ch_axis = 0
        self.register_buffer("weight_int8", T.tensor(np.zeros((num_embeddings, embedding_dim), np.int8), device="hip"))
        self.register_buffer("weight_scale", T.tensor(np.ones(num_embeddings, np.float32), device="hip"))
        self.register_buffer("weight_zero_point", T.tensor(np.zeros(num_embeddings, np.float32), device="hip"))

    def forward(self, x: Tensor, offsets: Tensor | None = None) -> Tensor:
        # lucid/nn/functional/sampling.py:442-517
        if self.mode not in _MODES:
            raise ValueError(f"embedding_bag: mode must be one of {sorted(_MODES)}, got {self.mode!r}")
        check_embedding_indices(x, self.num_embeddings, "embedding_bag")
        pad = -1 if self.padding_idx is None else int(self.padding_idx)
        if x.ndim == 2:
            bags, fixed, off_ptr, off64 = x.shape[0], x.shape[1], None, 0
        else:
            if offsets is None:
                raise ValueError("embedding_bag: offsets required for 1-D input")
            if not isinstance(offsets, Tensor) or offsets.device != "hip" or offsets.dtype not in (T.int32, T.int64):
                raise _C.DtypeMismatch("embedding_bag: offsets must be an int32 / int64 tensor on the 'hip' device")
            bags, fixed, off_ptr, off64 = offsets.numel, 0, offsets.data_ptr, int(offsets.dtype is T.int64)
        out = Tensor.empty((bags, self.embedding_dim), T.float32, "hip")
        _C.call("lq_embedding_bag_i8", self.weight_int8.data_ptr, self.weight_scale.data_ptr,
                self.weight_zero_point.data_ptr, self.num_embeddings, self.embedding_dim, x.data_ptr,
                int(x.dtype is T.int64), x.numel, off_ptr, off64, fixed, bags, _MODES[self.mode], pad,
                out.data_ptr, None)
        return out

    @classmethod
    def from_float(cls, mod) -> "EmbeddingBag":
        q = cls(mod.num_embeddings, mod.embedding_dim, mode=getattr(mod, "mode", "mean"),
                padding_idx=getattr(mod, "padding_idx", None))
        codes, scale, zero_point = _quantize_table(mod)
        q.register_buffer("weight_int8", codes)
        q.register_buffer("weight_scale", scale)
        q.register_buffer("weight_zero_point", zero_point)
        return q

    def extra_repr(self) -> str:
        return f"num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim}, mode={self.mode}"
