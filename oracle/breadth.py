"""CPU restatement of the quantized module breadth: int8 embedding tables, activations
that requantize their result, transposed convolution, the weight-only LSTM.

TEST INFRASTRUCTURE ONLY, like the rest of ``oracle/``.  numpy float32, plain loops
where the reference loops.

* ``embedding``      ``lucid/nn/quantized/sparse.py:128-134`` (dequantize the table,
                     ``F.embedding``) with ``CpuBackend.h:8970-9010`` (padding row = zeros)
* ``embedding_bag``  ``sparse.py:270-279`` with ``CpuBackend.h:5989-6088`` (bag bounds,
                     skipped ids, sum in index order, mean over the rows added, max from
                     the lowest float, an empty bag gives zeros)
* ``act``            ``CpuBackend.h:1049-1060`` sigmoid, ``:1722-1723`` leaky_relu,
                     ``:1783-1785`` elu, ``:2001-2002`` hard_sigmoid, ``:2064-2065``
                     hard_swish, tanh
* ``quantized_act``  ``lucid/nn/quantized/activation.py:44-53`` (activation, then
                     fake-quantize to the calibrated grid)
* ``lstm``           ``CpuBackend.h:13394-13519`` on dequantized weights
                     (``lucid/nn/quantized/dynamic/rnn.py``)
* ``qconv3d``        ``lucid/nn/quantized/conv.py:545-700`` (dequantize kernel, ``F.conv3d``,
                     bias, fake-quantize) in the integer formulation of the 2-d layer: taps
                     gathered with numpy slices, then the oracle's ``qlinear`` per group;
                     ``tests/test_oracle_breadth.py`` pins the gather and the group
                     bookkeeping against ``scipy.signal.correlate`` on the centred codes
* ``qconv_transpose3d``  ``lucid/nn/quantized/conv_transpose.py:484-640`` as ``qconv3d`` of the
                     zero-inserted codes with the flipped kernel; the same test file pins that
                     identity against the scatter definition of a transposed convolution

PARITY UNPINNED at the bit level for sigmoid, tanh, elu (the reference evaluates exp /
tanh through Accelerate's vForce, whose last-bit behaviour is not published) and for the
LSTM's float32 GEMMs (``cblas_sgemm`` accumulation order).  ``tests/test_oracle_breadth.py``
pins the formulas against float64 closed forms; hard_sigmoid, hard_swish, leaky_relu and
the embedding lookups are exact arithmetic and compared bit for bit.
"""

from __future__ import annotations

import numpy as np

import oracle as O

SIGMOID, HARDSWISH, HARDSIGMOID, TANH, ELU, LEAKY_RELU = range(6)


def dequantize_rows(codes, scale, zp):
    codes = np.asarray(codes)
    return ((codes.astype(np.float32) - np.asarray(zp, np.float32)[:, None]) *
            np.asarray(scale, np.float32)[:, None]).astype(np.float32)


def embedding(codes, scale, zp, idx, padding_idx=None):
    table = dequantize_rows(codes, scale, zp)
    idx = np.asarray(idx)
    out = table[idx.reshape(-1)].reshape(idx.shape + (table.shape[1],)).copy()
    if padding_idx is not None and padding_idx >= 0:
        out[idx == padding_idx] = 0.0
    return out


def embedding_bag(codes, scale, zp, idx, offsets=None, mode="mean", padding_idx=None):
    table = dequantize_rows(codes, scale, zp)
    num, D = table.shape
    idx = np.asarray(idx)
    if idx.ndim == 2:
        offsets = np.arange(0, idx.size, idx.shape[1])
        idx = idx.reshape(-1)
    offsets = np.asarray(offsets)
    B, n = len(offsets), idx.size
    pad = -1 if padding_idx is None else int(padding_idx)
    out = np.zeros((B, D), np.float32)
    for b in range(B):
        s = int(offsets[b])
        e = int(offsets[b + 1]) if b + 1 < B else n
        row = np.full(D, np.finfo(np.float32).min, np.float32) if mode == "max" else np.zeros(D, np.float32)
        count = 0
        for k in range(s, e):
            i = int(idx[k])
            if i == pad or i < 0 or i >= num:
                continue
            if mode == "max":
                row = np.where(table[i] > row, table[i], row)
            else:
                row = (row + table[i]).astype(np.float32)
            count += 1
        if mode == "max" and count == 0:
            row = np.zeros(D, np.float32)
        if mode == "mean" and count > 0:
            row = (row / np.float32(count)).astype(np.float32)
        out[b] = row
    return out


def act(kind, x, alpha=0.0):
    x = np.asarray(x, np.float32)
    one, alpha = np.float32(1.0), np.float32(alpha)
    with np.errstate(over="ignore"):
        if kind == SIGMOID:
            return (one / (one + np.exp(-x).astype(np.float32))).astype(np.float32)
        if kind in (HARDSWISH, HARDSIGMOID):
            t = ((x + np.float32(3.0)) / np.float32(6.0)).astype(np.float32)
            t = np.where(t < 0, np.float32(0.0), t)
            t = np.where(one < t, one, t).astype(np.float32)
            return (x * t).astype(np.float32) if kind == HARDSWISH else t
        if kind == TANH:
            return np.tanh(x).astype(np.float32)
        if kind == ELU:
            return np.where(x >= 0, x, alpha * (np.exp(x).astype(np.float32) - one)).astype(np.float32)
        if kind == LEAKY_RELU:
            return np.where(x >= 0, x, alpha * x).astype(np.float32)
    raise ValueError(kind)


def quantized_act(kind, x, alpha, S, Z, qmin, qmax):
    """Float output of ``_QuantizedActivation.forward``."""
    return O.fake_quantize(act(kind, x, alpha), S, Z, qmin, qmax)


def quantized_act_codes(kind, q, in_offset, s, z, alpha, S, Z, qmin, qmax, out_offset):
    """The same for an input carried as stored codes (``code + in_offset``), result as
    stored codes."""
    x = O.dequantize(np.asarray(q, np.int8), s, z, code_offset=in_offset)
    return O.quantize(act(kind, x, alpha), S, Z, qmin, qmax, code_offset=out_offset)


def lstm(x, h0, c0, w_ih, w_hh, b_ih, b_hh, w_hr=None, batch_sizes=None, reverse=False):
    """One layer, one direction, time-major ``x`` (T, B, I); returns (y, h_n, c_n).

    The recurrence of ``lstm_forward_train`` (CpuBackend.h:13394-13519): gates i, f, g, o;
    with ``w_hr`` (P, H) the step's output and next hidden state are the projection
    ``(o * tanh(c)) W_hr^T`` (lines 13503-13511).  ``batch_sizes`` (non-increasing, one per
    step) is the active-set schedule of a packed batch (lucid/nn/modules/rnn.py:585-650):
    at step t only the first ``batch_sizes[t]`` rows advance, the rest keep their state and
    their output row is zero.  ``reverse`` walks the steps from the last to the first."""
    x = np.asarray(x, np.float32)
    T, B, _ = x.shape
    H = c0.shape[-1]
    R = H if w_hr is None else w_hr.shape[0]
    h, c = np.asarray(h0, np.float32).copy(), np.asarray(c0, np.float32).copy()
    bias = (np.asarray(b_ih, np.float32) + np.asarray(b_hh, np.float32)).astype(np.float32)
    y = np.zeros((T, B, R), np.float32)
    sig = lambda v: (np.float32(1.0) / (np.float32(1.0) + np.exp(-v).astype(np.float32))).astype(np.float32)
    for t in (range(T - 1, -1, -1) if reverse else range(T)):
        n = B if batch_sizes is None else int(batch_sizes[t])
        if n == 0:
            continue
        raw = ((x[t, :n] @ w_ih.T).astype(np.float32) + (h[:n] @ w_hh.T).astype(np.float32)).astype(np.float32)
        raw = (raw + bias).astype(np.float32)
        i, f = sig(raw[:, :H]), sig(raw[:, H:2 * H])
        g, o = np.tanh(raw[:, 2 * H:3 * H]).astype(np.float32), sig(raw[:, 3 * H:])
        c[:n] = (f * c[:n] + i * g).astype(np.float32)
        hr = (o * np.tanh(c[:n]).astype(np.float32)).astype(np.float32)
        h[:n] = hr if w_hr is None else (hr @ np.asarray(w_hr, np.float32).T).astype(np.float32)
        y[t, :n] = h[:n]
    return y, h, c


def conv_transpose2d(x, w, bias, stride, padding, output_padding, dilation=(1, 1), groups=1):
    """Float64 scatter form of a transposed convolution: ``x`` (B, Cin, H, W), ``w``
    (Cin, Cout/groups, kh, kw)."""
    x = np.asarray(x, np.float64)
    w = np.asarray(w, np.float64)
    B, Cin, H, W = x.shape
    _, Cog, kh, kw = w.shape
    (sh, sw), (ph, pw), (oph, opw), (dh, dw) = stride, padding, output_padding, dilation
    OH = (H - 1) * sh - 2 * ph + dh * (kh - 1) + oph + 1
    OW = (W - 1) * sw - 2 * pw + dw * (kw - 1) + opw + 1
    full = np.zeros((B, Cog * groups, OH + 2 * ph, OW + 2 * pw), np.float64)
    cig = Cin // groups
    for g in range(groups):
        for ci in range(g * cig, (g + 1) * cig):
            for i in range(kh):
                for j in range(kw):
                    contrib = x[:, ci, :, :, None] * w[ci, :, i, j][None, None, None, :]  # B,H,W,Cog
                    full[:, g * Cog:(g + 1) * Cog, i * dh:i * dh + (H - 1) * sh + 1:sh,
                         j * dw:j * dw + (W - 1) * sw + 1:sw] += np.transpose(contrib, (0, 3, 1, 2))
    out = full[:, :, ph:ph + OH, pw:pw + OW]
    if bias is not None:
        out = out + np.asarray(bias, np.float64)[None, :, None, None]
    return out


def qconv3d(x, w, a_zp, a_scale, w_scale, stride=(1, 1, 1), pad=((0, 0),) * 3, dilation=(1, 1, 1), groups=1,
            bias=None, relu=False, **out):
    """Integer-formulation Conv3d.  ``x`` int8 stored codes (B, C, D, H, W); ``w`` int8
    (Cout, C/groups, KD, KH, KW); ``a_zp`` the input zero point as a stored code (what the
    padding holds); ``pad`` = ((lo, hi),) * 3; ``out``: the ``qlinear`` output arguments
    (``out_mode``, ``out_scale``, ...).  Returns (B, Cout, OD, OH, OW)."""
    import oracle as O
    x = np.asarray(x, np.int8)
    w = np.asarray(w, np.int8)
    B, C = x.shape[:2]
    Co, Cg = w.shape[:2]
    K3 = w.shape[2:]
    assert Cg * groups == C and Co % groups == 0
    xp = np.pad(x, ((0, 0), (0, 0), *pad), constant_values=np.int8(a_zp))
    outs = [(n - d * (k - 1) - 1) // s + 1 for n, k, s, d in zip(xp.shape[2:], K3, stride, dilation)]
    taps = []
    for kd in range(K3[0]):
        for kh in range(K3[1]):
            for kw in range(K3[2]):
                sl = tuple(slice(kk * d, kk * d + (o - 1) * s + 1, s)
                           for kk, d, o, s in zip((kd, kh, kw), dilation, outs, stride))
                taps.append(xp[(slice(None), slice(None), *sl)])          # (B, C, OD, OH, OW)
    cols = np.stack(taps, axis=0)                                          # (taps, B, C, OD, OH, OW)
    cols = np.transpose(cols, (1, 3, 4, 5, 0, 2))                          # (B, OD, OH, OW, taps, C)
    M = B * outs[0] * outs[1] * outs[2]
    Og = Co // groups
    parts = []
    for g in range(groups):
        a = np.ascontiguousarray(cols[..., g * Cg:(g + 1) * Cg]).reshape(M, -1)
        wg = w[g * Og:(g + 1) * Og].reshape(Og, Cg, -1)
        wg = np.ascontiguousarray(np.transpose(wg, (0, 2, 1))).reshape(Og, -1)   # k = tap * Cg + c
        ws = np.asarray(w_scale, np.float32)
        parts.append(O.qlinear(a, wg, a_zp, a_scale, ws[g * Og:(g + 1) * Og] if ws.ndim else ws,
                               bias=None if bias is None else np.asarray(bias)[g * Og:(g + 1) * Og],
                               relu=relu, **out))
    y = np.concatenate(parts, axis=1).reshape(B, *outs, Co)
    return np.ascontiguousarray(np.moveaxis(y, -1, 1))


def qconv_transpose3d(x, w, a_zp, a_scale, w_scale, stride=(1, 1, 1), padding=(0, 0, 0), output_padding=(0, 0, 0),
                      dilation=(1, 1, 1), groups=1, bias=None, **out):
    """Integer-formulation ConvTranspose3d.  ``x`` int8 stored codes (B, Cin, D, H, W); ``w``
    int8 (Cin, Cout/groups, KD, KH, KW); ``w_scale`` per output channel of a group (Cout/groups,),
    shared by the groups.  Zero-insert the codes (inserted codes = ``a_zp``), flip the kernel,
    swap its channel axes inside each group, convolve with stride 1 and padding
    ``dilation * (k - 1) - padding`` (``+ output_padding`` on the high side)."""
    x = np.asarray(x, np.int8)
    w = np.asarray(w, np.int8)
    B, Cin = x.shape[:2]
    K3 = w.shape[2:]
    spread = np.full((B, Cin, *[(n - 1) * s + 1 for n, s in zip(x.shape[2:], stride)]), np.int8(a_zp), np.int8)
    spread[(slice(None), slice(None), *[slice(None, None, s) for s in stride])] = x
    cig = Cin // groups
    wc = np.concatenate([np.transpose(w[g * cig:(g + 1) * cig, :, ::-1, ::-1, ::-1], (1, 0, 2, 3, 4))
                         for g in range(groups)], axis=0)                       # (Cout, Cin/groups, K3)
    lo = [d * (k - 1) - p for d, k, p in zip(dilation, K3, padding)]
    pad = tuple((l, l + op) for l, op in zip(lo, output_padding))
    return qconv3d(spread, wc, a_zp, a_scale, np.tile(np.asarray(w_scale, np.float32), groups), pad=pad,
                   dilation=dilation, groups=groups, bias=bias, **out)
