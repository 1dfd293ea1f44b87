"""Dynamic-quantized (weight-only int8) ``LSTM``
(``lucid/nn/quantized/dynamic/rnn.py:13-111``): every ``weight_*`` of the float LSTM is
stored as ``<name>_int8`` codes with a per-row ``<name>_scale`` (symmetric, zero point
0), the biases stay float; a forward decodes the weights and runs the float recurrence
(``CpuBackend.h:13394-13519``: gates i, f, g, o; ``raw = x W_ih^T + h W_hh^T + (b_ih +
b_hh)``).

On the device the input product of a layer is taken once over all time steps
(float32 MFMA GEMM), then each step is one recurrent GEMM and one gate kernel.
"""

from __future__ import annotations

import numpy as np

from .... import _C
from .... import _tensor as T
from ...._tensor import Tensor
from ....quantization._functional import dequantize, quantize
from ....quantization._qscheme import QDtype, per_channel_symmetric, qint8
from ...functional import linear_f32
from ...module import Module


class LSTM(Module):
    def __init__(self, input_size: int, hidden_size: int, num_layers: int = 1, bias: bool = True,
                 batch_first: bool = False, bidirectional: bool = False, proj_size: int = 0) -> None:
        super().__init__()
        self.input_size, self.hidden_size, self.num_layers = input_size, hidden_size, num_layers
        self.bias, self.batch_first, self.bidirectional = bias, batch_first, bidirectional
        self.proj_size = proj_size
        self._weight_names: list[str] = []
        self._bias_names: list[str] = []
        dirs = 2 if bidirectional else 1
        rec = proj_size if proj_size > 0 else hidden_size  # width of the state that re-enters the recurrence
        for k in range(num_layers):
            fan = input_size if k == 0 else rec * dirs
            for suffix in ("", "_reverse")[:dirs]:
                shapes = [(f"weight_ih_l{k}{suffix}", 4 * hidden_size, fan), (f"weight_hh_l{k}{suffix}", 4 * hidden_size, rec)]
                if proj_size > 0:
                    shapes.append((f"weight_hr_l{k}{suffix}", proj_size, hidden_size))
                for name, rows, cols in shapes:
                    self._weight_names.append(name)
                    self.register_buffer(name + "_int8", T.tensor(np.zeros((rows, cols), np.int8), device="hip"))
                    self.register_buffer(name + "_scale", T.tensor(np.ones(rows, np.float32), device="hip"))
                if bias:
                    for name in (f"bias_ih_l{k}{suffix}", f"bias_hh_l{k}{suffix}"):
                        self._bias_names.append(name)
                        self.register_buffer(name, T.tensor(np.zeros(4 * hidden_size, np.float32), device="hip"))

    def _weight(self, name: str) -> Tensor:
        codes, scale = getattr(self, name + "_int8"), getattr(self, name + "_scale")
        zp = T.tensor(np.zeros(scale.shape, np.float32), device="hip")
        return dequantize(codes, scale, zp, ch_axis=0)

    def forward(self, x, hx=None):
        """``x``: a float32 device tensor ``(T, B, I)`` / ``(B, T, I)``, or a ``PackedSequence``
        of one (``lucid/nn/modules/rnn.py:706-795``).  Packed input runs in packed (descending
        length) order: at step ``t`` only the first ``batch_sizes[t]`` rows advance, the others
        keep their state, which is why the final states hold every sequence's value at its own
        last step in either direction; outputs past a sequence's end are dropped by the
        repacking.  As in Lucid, a given ``hx`` is taken in packed order, and the returned
        states are put back into the caller's batch order."""
        from ...utils.rnn import PackedSequence
        packed = x if isinstance(x, PackedSequence) else None
        H, P, dirs = self.hidden_size, self.proj_size, 2 if self.bidirectional else 1
        R = P if P > 0 else H
        if packed is not None:
            data = packed.data
            if not isinstance(data, Tensor) or data.device != "hip" or data.dtype != T.float32:
                raise _C.DeviceMismatch("dynamic LSTM: packed data must be a float32 tensor on the 'hip' device")
            if data.ndim != 2 or data.shape[1] != self.input_size:
                raise _C.ShapeMismatch(f"dynamic LSTM: packed data must be (sum(batch_sizes), {self.input_size}), "
                                       f"got {data.shape}")
            batch_sizes = [int(v) for v in packed.batch_sizes.numpy().reshape(-1)]
            if sum(batch_sizes) != data.shape[0] or any(a < b for a, b in zip(batch_sizes, batch_sizes[1:])):
                raise ValueError("dynamic LSTM: batch_sizes must be non-increasing and sum to the packed length")
            Tn, Bn = len(batch_sizes), batch_sizes[0] if batch_sizes else 0
            # (T, B, I) in packed order, zeros past each sequence's end (rnn.py:40-80)
            x = Tensor.empty((Tn, Bn, self.input_size), T.float32, "hip")
            _C.call("lq_fill_bytes", x.data_ptr, 0, x.nbytes, None)
            off, rb = 0, self.input_size * 4
            for t, bs in enumerate(batch_sizes):
                _C.call("lq_d2d", x.data_ptr + t * Bn * rb, data.data_ptr + off * rb, bs * rb, None)
                off += bs
            batch_first = False
        else:
            if not isinstance(x, Tensor) or x.device != "hip" or x.dtype != T.float32:
                raise _C.DeviceMismatch("dynamic LSTM: input must be a float32 tensor on the 'hip' device")
            if x.ndim != 3 or x.shape[2] != self.input_size:
                raise _C.ShapeMismatch(f"dynamic LSTM: expected a 3-d input with {self.input_size} features, got {x.shape}")
            batch_first = self.batch_first
            Bn, Tn = (x.shape[0], x.shape[1]) if batch_first else (x.shape[1], x.shape[0])
            batch_sizes = [Bn] * Tn
        # row (t, b) of a (T, B, *) or (B, T, *) tensor: start of step t, row stride over b
        step_off = (lambda t, width: t * width) if batch_first else (lambda t, width: t * Bn * width)
        row_ld = (lambda width: Tn * width) if batch_first else (lambda width: width)
        n_state = self.num_layers * dirs
        if hx is None:
            h0 = c0 = None
        else:
            h0, c0 = hx
            if h0.shape != (n_state, Bn, R) or c0.shape != (n_state, Bn, H):
                raise _C.ShapeMismatch(f"dynamic LSTM: states must be {(n_state, Bn, R)} and {(n_state, Bn, H)}, "
                                       f"got {h0.shape} and {c0.shape}")
        h_n = Tensor.empty((n_state, Bn, R), T.float32, "hip")
        c_n = Tensor.empty((n_state, Bn, H), T.float32, "hip")
        ragged = any(bs != Bn for bs in batch_sizes)
        layer_in = x
        for k in range(self.num_layers):
            out_shape = (Bn, Tn, dirs * R) if batch_first else (Tn, Bn, dirs * R)
            y = Tensor.empty(out_shape, T.float32, "hip")
            if ragged:  # steps past a sequence's end stay zero
                _C.call("lq_fill_bytes", y.data_ptr, 0, y.nbytes, None)
            for d, suffix in enumerate(("", "_reverse")[:dirs]):
                w_ih, w_hh = self._weight(f"weight_ih_l{k}{suffix}"), self._weight(f"weight_hh_l{k}{suffix}")
                w_hr = self._weight(f"weight_hr_l{k}{suffix}") if P > 0 else None
                bias = None
                if self.bias:
                    b = getattr(self, f"bias_ih_l{k}{suffix}").numpy() + getattr(self, f"bias_hh_l{k}{suffix}").numpy()
                    bias = T.tensor(b.astype(np.float32), device="hip")
                gx = linear_f32(layer_in, w_ih)  # (.., .., 4H), same row order as layer_in
                idx = k * dirs + d
                h = Tensor.empty((Bn, R), T.float32, "hip")
                c = Tensor.empty((Bn, H), T.float32, "hip")
                for t_state, src, width in ((h, h0, R), (c, c0, H)):
                    if src is None:
                        _C.call("lq_fill_bytes", t_state.data_ptr, 0, Bn * width * 4, None)
                    else:
                        _C.call("lq_d2d", t_state.data_ptr, src.data_ptr + idx * Bn * width * 4, Bn * width * 4, None)
                h_raw = Tensor.empty((Bn, H), T.float32, "hip") if P > 0 else None
                for t in (range(Tn - 1, -1, -1) if d == 1 else range(Tn)):
                    bs = batch_sizes[t]
                    if bs == 0:
                        continue
                    gh = linear_f32(h.narrow_rows(bs), w_hh)
                    y_t = y.data_ptr + 4 * (step_off(t, dirs * R) + d * R)
                    if P == 0:
                        # h and c are updated in place (a gate element is read before it is written)
                        _C.call("lq_lstm_cell_f32", gx.data_ptr + 4 * step_off(t, 4 * H), row_ld(4 * H), gh.data_ptr,
                                bias.data_ptr if bias is not None else None, c.data_ptr, bs, H, h.data_ptr, c.data_ptr,
                                y_t, row_ld(dirs * R), None)
                    else:
                        # h_raw = o * tanh(c); the step's output and next state are its projection
                        # h_raw W_hr^T (CpuBackend.h:13503-13511)
                        _C.call("lq_lstm_cell_f32", gx.data_ptr + 4 * step_off(t, 4 * H), row_ld(4 * H), gh.data_ptr,
                                bias.data_ptr if bias is not None else None, c.data_ptr, bs, H, h_raw.data_ptr,
                                c.data_ptr, None, 0, None)
                        proj = linear_f32(h_raw.narrow_rows(bs), w_hr)
                        _C.call("lq_d2d", h.data_ptr, proj.data_ptr, bs * P * 4, None)
                        _C.call("lq_d2d_rows", y_t, row_ld(dirs * R) * 4, proj.data_ptr, P * 4, P * 4, bs, None)
                _C.call("lq_d2d", h_n.data_ptr + idx * Bn * R * 4, h.data_ptr, Bn * R * 4, None)
                _C.call("lq_d2d", c_n.data_ptr + idx * Bn * H * 4, c.data_ptr, Bn * H * 4, None)
            layer_in = y
        if packed is None:
            return layer_in, (h_n, c_n)
        # repack (rnn.py:83-98) and put the states back into the caller's batch order (rnn.py:137-150)
        out = Tensor.empty((sum(batch_sizes), dirs * R), T.float32, "hip")
        off, rb = 0, dirs * R * 4
        for t, bs in enumerate(batch_sizes):
            _C.call("lq_d2d", out.data_ptr + off * rb, layer_in.data_ptr + t * Bn * rb, bs * rb, None)
            off += bs
        if packed.unsorted_indices is not None:
            order = [int(v) for v in packed.unsorted_indices.numpy().reshape(-1)]
            if order != list(range(len(order))):
                def restore(state, width):
                    res = Tensor.empty(state.shape, T.float32, "hip")
                    for s_i in range(n_state):
                        for i, src in enumerate(order):
                            _C.call("lq_d2d", res.data_ptr + (s_i * Bn + i) * width * 4,
                                    state.data_ptr + (s_i * Bn + src) * width * 4, width * 4, None)
                    return res
                h_n, c_n = restore(h_n, R), restore(c_n, H)
        return PackedSequence(out, packed.batch_sizes, packed.sorted_indices, packed.unsorted_indices), (h_n, c_n)

    @classmethod
    def from_float(cls, mod, dtype: QDtype = qint8) -> "LSTM":
        from ....quantization.observer import PerChannelMinMaxObserver
        from ... import LSTM as FloatLSTM
        if not isinstance(mod, FloatLSTM):
            raise TypeError(f"dynamic LSTM.from_float expects an nn.LSTM, got {type(mod).__name__}")
        q = cls(mod.input_size, mod.hidden_size, mod.num_layers, mod.bias, mod.batch_first, mod.bidirectional,
                getattr(mod, "proj_size", 0))
        for name, param in mod.named_parameters():
            if name.startswith("weight"):
                obs = PerChannelMinMaxObserver(ch_axis=0, qscheme=per_channel_symmetric, qdtype=dtype)
                p = param.to("hip")
                obs(p)
                scale, zero_point = obs.calculate_qparams()
                q.register_buffer(name + "_int8", quantize(p, scale, zero_point, dtype, ch_axis=0))
                q.register_buffer(name + "_scale", scale.to("hip"))
            else:
                q.register_buffer(name, param.to("hip"))
        return q
