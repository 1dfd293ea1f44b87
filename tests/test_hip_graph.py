"""HIP-graph replay of a quantized forward equals the eager result on every
replay, with eager work and synchronisations in between, and the caching
allocator keeps graph-owned memory away from other tensors."""

import ctypes as C

import numpy as np
import pytest

import lucid_amd as L
import lucid_amd.nn.quantized as nnq
from lucid_amd import _C
import workloads as W

pytestmark = pytest.mark.gpu


def test_allocator_reuses_and_reports():
    _C.init()
    import gc
    gc.collect()
    _C.call("lq_empty_cache")                       # no cached block of this size left from earlier tests
    used0, res0 = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used0), C.byref(res0))
    a = L.Tensor.empty((1 << 20,), L.float32, "hip")
    p = a.data_ptr
    used1, res1 = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used1), C.byref(res1))
    assert used1.value >= used0.value + (4 << 20)
    del a
    b = L.Tensor.empty((1 << 20,), L.float32, "hip")
    assert b.data_ptr == p                          # the cached block came back
    _C.call("lq_memory_stats", C.byref(used1), C.byref(res1))
    del b
    _C.call("lq_empty_cache")
    used2, res2 = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used2), C.byref(res2))
    assert res2.value <= res1.value and used2.value <= used1.value
    with pytest.raises(ValueError):
        _C.call("lq_free", 0x1000)                  # not ours


def test_resnet50_graph_replay_matches_eager():
    model = W.QResNet50()
    rng = np.random.default_rng(0)
    batches = [rng.uniform(0, 1, (4, 3, 96, 96)).astype(np.float32) for _ in range(4)]
    eager = []
    for b in batches:
        eager.append(model(L.tensor(b, device="hip")).numpy())
    x = L.tensor(batches[0], device="hip")
    with L.graph.capture() as g:
        y = model(x)
    for rep in range(3):
        for i, b in enumerate(batches):
            x.copy_from(b)
            g.replay()
            # unrelated eager work and allocations between replays must not disturb the graph
            junk = L.tensor(rng.standard_normal(50000).astype(np.float32), device="hip")
            q = nnq.Quantize(L.tensor(np.float32(0.1), device="hip"),
                             L.tensor(np.float32(3.0), device="hip"))(junk)
            assert q._grid.codes.numpy().shape == (50000,)
            L.synchronize()
            assert np.array_equal(y.numpy(), eager[i]), (rep, i)
    g.destroy()
    # after destroy the eager path still works and memory went back to the pool
    assert np.array_equal(model(L.tensor(batches[1], device="hip")).numpy(), eager[1])


def test_capture_needs_a_created_stream():
    gid = C.c_int()
    with pytest.raises(ValueError):
        _C.call("lq_graph_begin", None, C.byref(gid))
