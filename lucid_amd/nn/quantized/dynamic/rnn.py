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
                 batch_first: bool = False, bidirectional: bool = False) -> None:
        super().__init__()
        self.input_size, self.hidden_size, self.num_layers = input_size, hidden_size, num_layers
        self.bias, self.batch_first, self.bidirectional = bias, batch_first, bidirectional
        self._weight_names: list[str] = []
        self._bias_names: list[str] = []
        dirs = 2 if bidirectional else 1
        for k in range(num_layers):
            fan = input_size if k == 0 else hidden_size * dirs
            for suffix in ("", "_reverse")[:dirs]:
                for name, cols in ((f"weight_ih_l{k}{suffix}", fan), (f"weight_hh_l{k}{suffix}", hidden_size)):
                    self._weight_names.append(name)
                    self.register_buffer(name + "_int8", T.tensor(np.zeros((4 * hidden_size, cols), np.int8),
                                                                  device="hip"))
                    self.register_buffer(name + "_scale", T.tensor(np.ones(4 * hidden_size, np.float32),
                                                                   device="hip"))
                if bias:
                    for name in (f"bias_ih_l{k}{suffix}", f"bias_hh_l{k}{suffix}"):
                        self._bias_names.append(name)
                        self.register_buffer(name, T.tensor(np.zeros(4 * hidden_size, np.float32), device="hip"))

    def _weight(self, name: str) -> Tensor:
        codes, scale = getattr(self, name + "_int8"), getattr(self, name + "_scale")
        zp = T.tensor(np.zeros(scale.shape, np.float32), device="hip")
        return dequantize(codes, scale, zp, ch_axis=0)

    def forward(self, x: Tensor, hx=None):
        if not isinstance(x, Tensor):
            raise NotImplementedError("dynamic LSTM on hip: PackedSequence input is not supported")
        if x.device != "hip" or x.dtype != T.float32:
            raise _C.DeviceMismatch("dynamic LSTM: input must be a float32 tensor on the 'hip' device")
        if x.ndim != 3 or x.shape[2] != self.input_size:
            raise _C.ShapeMismatch(f"dynamic LSTM: expected a 3-d input with {self.input_size} features, got {x.shape}")
        H, dirs = self.hidden_size, 2 if self.bidirectional else 1
        Bn, Tn = (x.shape[0], x.shape[1]) if self.batch_first else (x.shape[1], x.shape[0])
        # row (t, b) of a (T, B, *) or (B, T, *) tensor: start of step t, row stride over b
        step_off = (lambda t, width: t * width) if self.batch_first else (lambda t, width: t * Bn * width)
        row_ld = (lambda width: Tn * width) if self.batch_first else (lambda width: width)
        n_state = self.num_layers * dirs
        if hx is None:
            h0 = c0 = None
        else:
            h0, c0 = hx
            for s in (h0, c0):
                if s.shape != (n_state, Bn, H):
                    raise _C.ShapeMismatch(f"dynamic LSTM: state must be {(n_state, Bn, H)}, got {s.shape}")
        h_n = Tensor.empty((n_state, Bn, H), T.float32, "hip")
        c_n = Tensor.empty((n_state, Bn, H), T.float32, "hip")
        layer_in = x
        for k in range(self.num_layers):
            out_shape = (Bn, Tn, dirs * H) if self.batch_first else (Tn, Bn, dirs * H)
            y = Tensor.empty(out_shape, T.float32, "hip")
            for d, suffix in enumerate(("", "_reverse")[:dirs]):
                w_ih, w_hh = self._weight(f"weight_ih_l{k}{suffix}"), self._weight(f"weight_hh_l{k}{suffix}")
                bias = None
                if self.bias:
                    b = getattr(self, f"bias_ih_l{k}{suffix}").numpy() + getattr(self, f"bias_hh_l{k}{suffix}").numpy()
                    bias = T.tensor(b.astype(np.float32), device="hip")
                gx = linear_f32(layer_in, w_ih)  # (.., .., 4H), same row order as layer_in
                idx = k * dirs + d
                state_bytes = Bn * H * 4
                h = Tensor.empty((Bn, H), T.float32, "hip")
                c = Tensor.empty((Bn, H), T.float32, "hip")
                for t_state, src in ((h, h0), (c, c0)):
                    if src is None:
                        _C.call("lq_fill_bytes", t_state.data_ptr, 0, state_bytes, None)
                    else:
                        _C.call("lq_d2d", t_state.data_ptr, src.data_ptr + idx * state_bytes, state_bytes, None)
                steps = range(Tn - 1, -1, -1) if d == 1 else range(Tn)
                for t in steps:
                    gh = linear_f32(h, w_hh)
                    # h and c are updated in place (a gate element is read before it is written);
                    # the last step writes the final state
                    last = t == (0 if d == 1 else Tn - 1)
                    h_dst = h_n.data_ptr + idx * state_bytes if last else h.data_ptr
                    c_dst = c_n.data_ptr + idx * state_bytes if last else c.data_ptr
                    _C.call("lq_lstm_cell_f32", gx.data_ptr + 4 * step_off(t, 4 * H), row_ld(4 * H), gh.data_ptr,
                            bias.data_ptr if bias is not None else None, c.data_ptr, Bn, H, h_dst, c_dst,
                            y.data_ptr + 4 * (step_off(t, dirs * H) + d * H), row_ld(dirs * H), None)
                if Tn == 0:
                    _C.call("lq_d2d", h_n.data_ptr + idx * state_bytes, h.data_ptr, state_bytes, None)
                    _C.call("lq_d2d", c_n.data_ptr + idx * state_bytes, c.data_ptr, state_bytes, None)
            layer_in = y
        return layer_in, (h_n, c_n)

    @classmethod
    def from_float(cls, mod, dtype: QDtype = qint8) -> "LSTM":
        from ....quantization.observer import PerChannelMinMaxObserver
        from ... import LSTM as FloatLSTM
        if not isinstance(mod, FloatLSTM):
            raise TypeError(f"dynamic LSTM.from_float expects an nn.LSTM, got {type(mod).__name__}")
        q = cls(mod.input_size, mod.hidden_size, mod.num_layers, mod.bias, mod.batch_first, mod.bidirectional)
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
