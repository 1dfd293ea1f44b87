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


@pytest.mark.parametrize("batch,parts", [(6, 2), (7, 3), (4, 4)])
def test_batch_split_replay_on_several_streams_matches_eager(batch, parts):
    """graph.capture_split: the forward captured once per slice of the batch, as parallel branches of
    one graph - the concatenated result equals one eager forward of the whole batch, replay
    after replay, with eager work between the replays and with new input in the same buffer."""
    model = W.QResNet50()
    rng = np.random.default_rng(batch)
    batches = [rng.uniform(0, 1, (batch, 3, 64, 64)).astype(np.float32) for _ in range(3)]
    eager = [model(L.tensor(b, device="hip")).numpy() for b in batches]
    x = L.tensor(batches[0], device="hip")
    bounds = [batch * i // parts for i in range(parts + 1)]
    for lo, hi in zip(bounds[:-1], bounds[1:]):
        model(x.row_range(lo, hi))  # every slice size once, eagerly
    sg = L.graph.capture_split(model, x, parts)
    assert sg.branches == parts and sg.output.shape == eager[0].shape
    for rep in range(2):
        for i, b in enumerate(batches):
            x.copy_from(b)
            sg.replay()
            junk = L.tensor(rng.standard_normal(30000).astype(np.float32), device="hip")
            assert np.isfinite(junk.numpy()).all()
            L.synchronize()
            assert np.array_equal(sg.output.numpy(), eager[i]), (rep, i)
    sg.destroy()
    assert np.array_equal(model(L.tensor(batches[1], device="hip")).numpy(), eager[1])


def test_capture_needs_a_created_stream():
    gid = C.c_int()
    with pytest.raises(ValueError):
        _C.call("lq_graph_begin", None, C.byref(gid))


def _stats():
    used, res = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used), C.byref(res))
    return used.value, res.value


def test_scratch_growth_after_capture_keeps_the_graph_valid():
    """A graph bakes the address of its stream's scratch into its kernel nodes.  A later call
    on the same stream that needs more scratch must not free that block under the graph."""
    _C.init()
    rng = np.random.default_rng(3)
    n = 1 << 22
    x = L.tensor(rng.standard_normal(n).astype(np.float32), device="hip")
    mn = L.Tensor.empty((1,), L.float32, "hip")
    mx = L.Tensor.empty((1,), L.float32, "hip")
    stream = C.c_void_p()
    _C.call("lq_stream_create", C.byref(stream))
    gid = C.c_int()
    _C.call("lq_sync", None)
    _C.call("lq_graph_begin", stream, C.byref(gid))
    try:
        # per-tensor min / max of 4 M elements: two stages, partial results in the stream's scratch
        _C.call("lq_minmax", x.data_ptr, 1, 1, n, mn.data_ptr, mx.data_ptr, stream)
    finally:
        _C.call("lq_graph_end", stream, gid.value)
    # eager work on the same stream that outgrows the 4 MiB scratch: the group-wise matmul with
    # M > 64 decodes its weight into N * K floats of scratch (16 MiB here)
    M, N, K = 65, 4096, 1024
    xs = L.tensor(np.zeros((M, K), np.float32), device="hip")
    packed = L.tensor(np.zeros((N, K // 4), np.int32), device="hip")
    sc = L.tensor(np.ones((N, K // 64), np.float32), device="hip")
    bi = L.tensor(np.zeros((N, K // 64), np.float32), device="hip")
    out = L.Tensor.empty((M, N), L.float32, "hip")
    _C.call("lq_wq_matmul", xs.data_ptr, packed.data_ptr, sc.data_ptr, bi.data_ptr, M, N, K, 64, 8,
            out.data_ptr, stream)
    _C.call("lq_sync", stream)
    for rep in range(3):
        data = rng.standard_normal(n).astype(np.float32) * (rep + 1)
        x.copy_from(data)
        _C.call("lq_graph_launch", gid.value, stream)
        _C.call("lq_sync", stream)
        assert mn.numpy()[0] == data.min() and mx.numpy()[0] == data.max(), rep
        # and once more with eager scratch use on the stream between the replays
        _C.call("lq_wq_matmul", xs.data_ptr, packed.data_ptr, sc.data_ptr, bi.data_ptr, M, N, K, 64, 8,
                out.data_ptr, stream)
    _C.call("lq_graph_destroy", gid.value)
    _C.call("lq_stream_destroy", stream)


def test_tensor_that_outlives_its_graph_keeps_its_memory():
    """Blocks allocated during capture go back to the pool at destroy only if their owner has
    freed them; a result tensor still alive keeps its block to itself."""
    import gc
    _C.init()
    gc.collect()
    _C.call("lq_empty_cache")  # so that the only cached block after destroy is the one released by it
    x = L.tensor(np.arange(4096, dtype=np.float32), device="hip")
    with L.graph.capture() as g:
        y = L.Tensor.empty((4096,), L.float32, "hip")
        _C.call("lq_relu_f32", x.data_ptr, y.data_ptr, 4096, None)
        tmp = L.Tensor.empty((4096,), L.float32, "hip")  # dies before the graph does
        _C.call("lq_relu_f32", x.data_ptr, tmp.data_ptr, 4096, None)
        tmp_ptr = tmp.data_ptr
        del tmp
    g.replay()
    L.synchronize()
    g.destroy()
    fresh = [L.Tensor.empty((4096,), L.float32, "hip") for _ in range(8)]
    ptrs = [t.data_ptr for t in fresh]
    assert y.data_ptr not in ptrs            # still owned by y
    assert tmp_ptr in ptrs                   # its owner was gone: released with the graph
    for t in fresh:
        t.copy_from(np.full(4096, -1.0, np.float32))
    L.synchronize()
    assert np.array_equal(y.numpy(), np.arange(4096, dtype=np.float32))
    used_before = _stats()[0]
    del y
    assert _stats()[0] < used_before         # y's own free released the block


def test_failed_capture_releases_its_blocks():
    import gc
    _C.init()
    gc.collect()
    x = L.tensor(np.ones(1 << 16, np.float32), device="hip")
    used0 = _stats()[0]
    with pytest.raises(RuntimeError, match="boom"):
        with L.graph.capture():
            t = L.Tensor.empty((1 << 16,), L.float32, "hip")
            _C.call("lq_relu_f32", x.data_ptr, t.data_ptr, 1 << 16, None)
            raise RuntimeError("boom")
    del t
    gc.collect()
    assert _stats()[0] == used0
    # and the library still captures and replays afterwards
    with L.graph.capture() as g:
        y = L.Tensor.empty((1 << 16,), L.float32, "hip")
        _C.call("lq_relu_f32", x.data_ptr, y.data_ptr, 1 << 16, None)
    g.replay()
    L.synchronize()
    assert np.all(y.numpy() == 1.0)
    g.destroy()


def test_failed_split_capture_releases_its_blocks_and_streams():
    """capture_split whose forward raises on the second slice (a branch stream has joined the
    capture and is never joined back): the error reaches the caller, the blocks allocated during
    the capture are released, and a following capture_split works."""
    import gc
    _C.init()
    gc.collect()
    x = L.tensor(np.arange(8 * 4096, dtype=np.float32).reshape(8, 4096) - 9000.0, device="hip")
    calls = []

    def relu(xs, fail_on=None):
        calls.append(xs.shape[0])
        if fail_on is not None and len(calls) == fail_on:
            raise RuntimeError("boom")
        y = L.Tensor.empty(xs.shape, L.float32, "hip")
        _C.call("lq_relu_f32", xs.data_ptr, y.data_ptr, xs.numel, None)
        return y

    used0 = _stats()[0]
    with pytest.raises(RuntimeError, match="boom"):
        L.graph.capture_split(lambda xs: relu(xs, fail_on=2), x, 2)
    gc.collect()
    assert _stats()[0] == used0
    assert _C.current_stream() is None
    calls.clear()
    sg = L.graph.capture_split(relu, x, 3)
    assert calls == [2, 3, 3]
    sg.replay()
    L.synchronize()
    assert np.array_equal(sg.output.numpy(), np.maximum(x.numpy(), 0.0))
    sg.destroy()


def test_vit_b16_batch64_graph_replay_matches_eager():
    """The serving configuration of the ViT bench: a captured forward of ViT-B/16 at batch 64
    gives the eager logits bit for bit on every replay, for several batches, with eager work
    and synchronisations in between (the dynamic quantizers' ranges live on the device, so
    nothing in the forward talks to the host)."""
    model = W.QViT(W.VIT_B16, seed=2)
    rng = np.random.default_rng(9)
    batches = [rng.uniform(0, 1, (64, 3, 224, 224)).astype(np.float32) for _ in range(3)]
    x = L.tensor(batches[0], device="hip")
    eager = []
    for b in batches:
        x.copy_from(b)
        eager.append(model(x).numpy())
    assert not np.array_equal(eager[0], eager[1])
    with L.graph.capture() as g:
        y = model(x)
    for rep in range(2):
        for i, b in enumerate(batches):
            x.copy_from(b)
            g.replay()
            junk = model.blocks[0].fc1(L.tensor(rng.standard_normal((7, 768)).astype(np.float32), device="hip"))
            L.synchronize()
            assert junk.shape == (7, 3072)
            assert np.array_equal(y.numpy().view(np.uint32), eager[i].view(np.uint32)), (rep, i)
    g.destroy()
    x.copy_from(batches[2])
    assert np.array_equal(model(x).numpy().view(np.uint32), eager[2].view(np.uint32))
