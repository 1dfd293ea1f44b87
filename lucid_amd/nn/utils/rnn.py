"""Variable-length batches for recurrent layers (``lucid/nn/utils/rnn.py``):
``PackedSequence`` and its pack / pad helpers.  The index bookkeeping is small host-side
metadata; the feature rows move with pitched device copies when the tensor lives on
``"hip"`` and with numpy when it lives on the host."""

from __future__ import annotations

from typing import NamedTuple

import numpy as np

from ... import _C
from ... import _tensor as T
from ..._tensor import Tensor


class PackedSequence(NamedTuple):
    """``data`` (sum(batch_sizes), *feat) walks time-major over the sequences in descending
    length order; ``batch_sizes[t]`` sequences are still running at step ``t``
    (``rnn.py:54-105``)."""

    data: Tensor
    batch_sizes: Tensor
    sorted_indices: Tensor | None
    unsorted_indices: Tensor | None


def _ints(t) -> list[int]:
    if isinstance(t, Tensor):
        return [int(v) for v in t.numpy().reshape(-1)]
    return [int(v) for v in t]


def _row_bytes(t: Tensor, from_axis: int) -> int:
    return int(np.prod(t.shape[from_axis:], dtype=np.int64)) * t.dtype.itemsize


def pack_padded_sequence(input: Tensor, lengths, batch_first: bool = False,  # noqa: A002 - Lucid's name
                         enforce_sorted: bool = True) -> PackedSequence:
    """``rnn.py:108-215``."""
    Tn, Bn = (input.shape[1], input.shape[0]) if batch_first else (input.shape[0], input.shape[1])
    feat = tuple(input.shape[2:])
    lens = _ints(lengths)
    if len(lens) != Bn:
        raise _C.ShapeMismatch(f"pack_padded_sequence: {len(lens)} lengths for a batch of {Bn}")
    order = sorted(range(Bn), key=lambda i: -lens[i])
    inverse = [0] * Bn
    for new, orig in enumerate(order):
        inverse[orig] = new
    if enforce_sorted:
        if any(lens[i] < lens[i + 1] for i in range(Bn - 1)):
            raise ValueError("pack_padded_sequence: sequences must be sorted by length in descending order "
                             "or pass enforce_sorted=False.")
        rows = list(range(Bn))
    else:
        rows = order
    slens = [lens[i] for i in rows]
    batch_sizes = []
    for t in range(Tn):
        bs = sum(1 for v in slens if v > t)
        if bs == 0:
            break
        batch_sizes.append(bs)
    total = sum(batch_sizes)
    if input.device == "cpu":
        a = input.numpy()
        tm = np.swapaxes(a, 0, 1) if batch_first else a
        data = T.tensor(np.concatenate([tm[t, rows[:bs]] for t, bs in enumerate(batch_sizes)], axis=0)
                        if batch_sizes else np.zeros((0, *feat), a.dtype))
    else:
        data = Tensor.empty((total, *feat), input.dtype, "hip")
        rb = _row_bytes(input, 2)
        # address of row (t, b) of the padded tensor
        t_stride, b_stride = (rb, Tn * rb) if batch_first else (Bn * rb, rb)
        off = 0
        for t, bs in enumerate(batch_sizes):
            if rows[:bs] == list(range(bs)):
                _C.call("lq_d2d_rows", data.data_ptr + off * rb, rb, input.data_ptr + t * t_stride, b_stride, rb, bs,
                        None)
            else:
                for j in range(bs):
                    _C.call("lq_d2d", data.data_ptr + (off + j) * rb, input.data_ptr + t * t_stride + rows[j] * b_stride,
                            rb, None)
            off += bs
    i64 = lambda v: T.tensor(np.asarray(v, np.int64))
    return PackedSequence(data, i64(batch_sizes), i64(order), i64(inverse))


def pad_packed_sequence(sequence: PackedSequence, batch_first: bool = False, padding_value: float = 0.0,
                        total_length: int | None = None) -> tuple[Tensor, Tensor]:
    """``rnn.py:218-323``: the padded batch in the caller's original order, and the lengths."""
    data = sequence.data
    batch_sizes = _ints(sequence.batch_sizes)
    Tn, Bn = len(batch_sizes), (batch_sizes[0] if batch_sizes else 0)
    if total_length is not None and total_length > Tn:
        Tn = total_length
    feat = tuple(data.shape[1:])
    lens = [sum(1 for bs in batch_sizes if bs > b) for b in range(Bn)]
    order = _ints(sequence.unsorted_indices) if sequence.unsorted_indices is not None else list(range(Bn))
    # original row i sits at packed position order[i]
    shape = (Bn, Tn, *feat) if batch_first else (Tn, Bn, *feat)
    if data.device == "cpu":
        a = data.numpy()
        tm = np.full((Tn, Bn, *feat), padding_value, a.dtype)
        off = 0
        for t, bs in enumerate(batch_sizes):
            tm[t, :bs] = a[off:off + bs]
            off += bs
        tm = tm[:, order]
        out = T.tensor(np.ascontiguousarray(np.swapaxes(tm, 0, 1) if batch_first else tm))
    else:
        if padding_value == 0.0:
            out = Tensor.empty(shape, data.dtype, "hip")
            _C.call("lq_fill_bytes", out.data_ptr, 0, out.nbytes, None)
        else:
            out = T.tensor(np.full(shape, padding_value, data.dtype.np), device="hip")
        rb = _row_bytes(data, 1)
        t_stride, b_stride = (rb, Tn * rb) if batch_first else (Bn * rb, rb)
        position = [0] * Bn  # packed position -> original row
        for orig, pos in enumerate(order):
            position[pos] = orig
        off = 0
        for t, bs in enumerate(batch_sizes):
            if position[:bs] == list(range(bs)):
                _C.call("lq_d2d_rows", out.data_ptr + t * t_stride, b_stride, data.data_ptr + off * rb, rb, rb, bs, None)
            else:
                for j in range(bs):
                    _C.call("lq_d2d", out.data_ptr + t * t_stride + position[j] * b_stride,
                            data.data_ptr + (off + j) * rb, rb, None)
            off += bs
    return out, T.tensor(np.asarray([lens[order[i]] for i in range(Bn)], np.int64))


def pad_sequence(sequences, batch_first: bool = False, padding_value: float = 0.0) -> Tensor:
    """Stack host sequences ``(L_i, *feat)`` into ``(T_max, B, *feat)`` (``rnn.py:326-396``)."""
    arrs = [s.numpy() for s in sequences]
    Tn = max(a.shape[0] for a in arrs)
    out = np.full((Tn, len(arrs), *arrs[0].shape[1:]), padding_value, arrs[0].dtype)
    for b, a in enumerate(arrs):
        out[:a.shape[0], b] = a
    res = T.tensor(np.ascontiguousarray(np.swapaxes(out, 0, 1) if batch_first else out))
    return res.to(sequences[0].device) if sequences[0].device != "cpu" else res


def pack_sequence(sequences, enforce_sorted: bool = True) -> PackedSequence:
    """``pad_sequence`` followed by ``pack_padded_sequence`` (``rnn.py:399-460``)."""
    lengths = [int(s.shape[0]) for s in sequences]
    return pack_padded_sequence(pad_sequence(sequences), lengths, enforce_sorted=enforce_sorted)
