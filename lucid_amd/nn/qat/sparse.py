"""QAT ``Embedding`` (``lucid/nn/qat/sparse.py:21-160``): the table is fake-quantized on every
forward, then looked up; there is no activation observer (a gather of rows that lie on the
grid lies on the grid)."""

from __future__ import annotations

from ... import _C
from ... import _tensor as T
from ..._tensor import Tensor
from .. import Embedding as _FloatEmbedding


class Embedding(_FloatEmbedding):
    def __init__(self, num_embeddings: int, embedding_dim: int, padding_idx: int | None = None, *,
                 qconfig=None) -> None:
        super().__init__(num_embeddings, embedding_dim, padding_idx)
        if qconfig is None:
            raise ValueError("qat.Embedding requires a qconfig")
        self.qconfig = qconfig
        self.weight_fake_quant = qconfig.weight()

    def forward(self, x: Tensor) -> Tensor:
        """``F.embedding(x, fake_quant(weight))``: a gather of fake-quantized rows, which is the
        dequantizing gather of their codes - (c - z) * s is evaluated for the rows that are
        looked up instead of for the whole table."""
        from ...quantization._functional import quantize
        from ..quantized.sparse import check_embedding_indices
        w = self.weight if self.weight.device == "hip" else self.weight.to("hip")
        fq = self.weight_fake_quant
        fq(w)  # observe (and, like any FakeQuantize call, refresh the qparams)
        scale, zero_point = fq.calculate_qparams()
        if fq.ch_axis not in (0, None) or fq.qdtype.storage != "int8":
            raise NotImplementedError("qat.Embedding: the weight FakeQuantize must be per-row or per-tensor int8")
        codes = quantize(w, scale, zero_point, fq.qdtype, ch_axis=fq.ch_axis)
        if fq.ch_axis is None:
            import numpy as np
            scale = T.tensor(np.full(self.num_embeddings, scale.item(), np.float32), device="hip")
            zero_point = T.tensor(np.full(self.num_embeddings, zero_point.item(), np.float32), device="hip")
        check_embedding_indices(x, self.num_embeddings, "embedding")
        out = Tensor.empty((*x.shape, self.embedding_dim), T.float32, "hip")
        pad = -1 if self.padding_idx is None else int(self.padding_idx)
        _C.call("lq_embedding_i8", codes.data_ptr, scale.to("hip").data_ptr, zero_point.to("hip").data_ptr,
                self.num_embeddings, self.embedding_dim, x.data_ptr, int(x.dtype is T.int64), x.numel, pad,
                out.data_ptr, None)
        return out

    @classmethod
    def from_float(cls, mod) -> "Embedding":
        qat = cls(mod.num_embeddings, mod.embedding_dim, padding_idx=mod.padding_idx, qconfig=mod.qconfig)
        qat.register_buffer("weight", mod.weight.to("hip"))
        return qat
