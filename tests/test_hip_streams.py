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


def test_fork_and_join_with_events_on_non_blocking_streams():
    """lq_stream_create_nonblocking + lq_event_record / lq_stream_wait_event: work forked from the
    default stream onto two streams that do not synchronise with it implicitly, joined back by
    events - the consumer on the default stream sees both results."""
    _C.init()
    rng = np.random.default_rng(5)
    n = 1 << 20
    x = L.tensor(rng.standard_normal(2 * n).astype(np.float32), device="hip")
    y = L.Tensor.empty((2 * n,), L.float32, "hip")
    streams, joins = [], []
    for _ in range(2):
        s, e = C.c_void_p(), C.c_void_p()
        _C.call("lq_stream_create_nonblocking", C.byref(s))
        _C.call("lq_event_create", C.byref(e))
        streams.append(s)
        joins.append(e)
    fork = C.c_void_p()
    _C.call("lq_event_create", C.byref(fork))
    try:
        for rep in range(3):
            x.copy_from(rng.standard_normal(2 * n).astype(np.float32))   # on the default stream
            _C.call("lq_event_record", fork, None)
            for i, (s, e) in enumerate(zip(streams, joins)):
                _C.call("lq_stream_wait_event", s, fork)
                _C.call("lq_relu_f32", x.data_ptr + 4 * n * i, y.data_ptr + 4 * n * i, n, s)
                _C.call("lq_event_record", e, s)
            for e in joins:
                _C.call("lq_stream_wait_event", None, e)
            z = L.Tensor.empty((2 * n,), L.float32, "hip")
            _C.call("lq_add_f32", y.data_ptr, y.data_ptr, z.data_ptr, 2 * n, None)  # consumer on the default stream
            assert np.array_equal(z.numpy(), 2 * np.maximum(x.numpy(), 0.0)), rep
    finally:
        L.synchronize()
        for s in streams:
            _C.call("lq_stream_destroy", s)
        for e in [fork, *joins]:
            _C.call("lq_event_destroy", e)
    with pytest.raises(ValueError, match="event is NULL"):
        _C.call("lq_stream_wait_event", None, None)
