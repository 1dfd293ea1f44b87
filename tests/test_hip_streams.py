"""Calls that overlap on two streams do not share library scratch: a split-K Linear and a
two-stage min / max issued alternately on two streams give the bits of the same calls run
one after the other (Lucid's dispatcher is concurrent-safe, ``Dispatcher.h:49-52``)."""

import ctypes as C

import numpy as np
import pytest

import lucid_amd as L
import oracle as O
from lucid_amd import _C, _ops

pytestmark = pytest.mark.gpu


def _linear(a, w, cfg):
    return _ops.qlinear_i8(a, w, out_mode=_ops.OUT_ACC_I32, path=_ops.PATH_TILE, tile_config=cfg)


def test_two_streams_share_no_scratch():
    _C.init()
    rng = np.random.default_rng(11)
    # few tiles, long K: the stream-K schedule splits K between blocks and exchanges partial sums
    # through the stream's slabs and arrival counters
    shapes = [(256, 256, 8192), (128, 384, 4096)]
    cfg = 5 | (2 << 8)
    ops = []
    for M, N, K in shapes:
        a = rng.integers(-128, 128, (M, K), dtype=np.int8)
        w = rng.integers(-128, 128, (N, K), dtype=np.int8)
        ops.append((L.tensor(a, device="hip"), L.tensor(w, device="hip"), O.igemm(a, w)))
    xs = [rng.standard_normal(1 << 21).astype(np.float32) * (i + 1) for i in range(2)]
    xd = [L.tensor(x, device="hip") for x in xs]
    streams = []
    for _ in range(2):
        s = C.c_void_p()
        _C.call("lq_stream_create", C.byref(s))
        streams.append(s)
    L.synchronize()
    prev = _C.current_stream()
    try:
        outs, ranges = [[], []], [[], []]
        for rep in range(6):
            for i in (0, 1):
                _C.set_current_stream(streams[i])
                a, w, _ = ops[i]
                outs[i].append(_linear(a, w, cfg))
                mn = L.Tensor.empty((1,), L.float32, "hip")
                mx = L.Tensor.empty((1,), L.float32, "hip")
                _C.call("lq_minmax", xd[i].data_ptr, 1, 1, xs[i].size, mn.data_ptr, mx.data_ptr, None)
                ranges[i].append((mn, mx))
        for s in streams:
            _C.call("lq_sync", s)
    finally:
        _C.set_current_stream(prev)
    for i in (0, 1):
        for y in outs[i]:
            assert np.array_equal(y.numpy(), ops[i][2]), i
        for mn, mx in ranges[i]:
            assert mn.numpy()[0] == xs[i].min() and mx.numpy()[0] == xs[i].max(), i
    for s in streams:
        _C.call("lq_stream_destroy", s)
