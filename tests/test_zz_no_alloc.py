"""``lq_minmax_noalloc``: the entry point that allocates nothing gives the bits of
``lq_minmax`` on two calls in a row (the second on a smaller input, so stale partial
results of the first are still in the static scratch), for every launch route, and
refuses what does not fit its scratch."""

import ctypes as C

import numpy as np
import pytest

import lucid_amd as L
import oracle as O
from lucid_amd import _C

pytestmark = pytest.mark.gpu


def _both(x, outer, Cn, inner):
    """(mn, mx) of lq_minmax and of lq_minmax_noalloc as uint32 bit patterns."""
    xd = L.tensor(x, device="hip")
    out = []
    for name in ("lq_minmax", "lq_minmax_noalloc"):
        mn = L.Tensor.empty((Cn,), L.float32, "hip")
        mx = L.Tensor.empty((Cn,), L.float32, "hip")
        _C.call(name, xd.data_ptr, outer, Cn, inner, mn.data_ptr, mx.data_ptr, None)
        out.append((mn.numpy().view(np.uint32).copy(), mx.numpy().view(np.uint32).copy()))
    return out


CASES = [
    # (outer, C, inner) of the first call, then of the smaller second call
    ((1, 1, 1 << 22), (1, 1, 300_000)),          # per tensor: many slices, partials in the scratch
    ((1, 16, 1 << 18), (1, 5, 70_000)),          # per channel, contiguous runs, split channels
    ((4096, 512, 1), (700, 96, 1)),              # channel-last: the column route
    ((3, 4096, 257), (2, 33, 65)),               # one block per channel, odd sizes (no partials)
]


@pytest.mark.parametrize("first,second", CASES)
def test_noalloc_equals_minmax_twice_in_a_row(first, second):
    _C.init()
    rng = np.random.default_rng(7)
    for outer, Cn, inner in (first, second):
        x = rng.standard_normal(outer * Cn * inner).astype(np.float32)
        x[rng.integers(0, x.size, 16)] *= 50.0
        (mn0, mx0), (mn1, mx1) = _both(x, outer, Cn, inner)
        assert np.array_equal(mn0, mn1) and np.array_equal(mx0, mx1), (outer, Cn, inner)
        omn, omx = O.minmax(x.reshape(outer, Cn, inner), ch_axis=1) if Cn > 1 else O.minmax(x)
        assert np.array_equal(np.asarray(omn, np.float32).reshape(-1).view(np.uint32), mn1)
        assert np.array_equal(np.asarray(omx, np.float32).reshape(-1).view(np.uint32), mx1)


def test_noalloc_propagates_nan_and_handles_empty():
    _C.init()
    x = np.arange(1 << 20, dtype=np.float32)
    x[12345] = np.nan
    (mn0, mx0), (mn1, mx1) = _both(x, 1, 1, x.size)
    assert np.isnan(mn1.view(np.float32)).all() and np.isnan(mx1.view(np.float32)).all()
    assert np.isnan(mn0.view(np.float32)).all()
    mn = L.Tensor.empty((3,), L.float32, "hip")
    mx = L.Tensor.empty((3,), L.float32, "hip")
    _C.call("lq_minmax_noalloc", None, 0, 3, 5, mn.data_ptr, mx.data_ptr, None)
    assert np.all(mn.numpy() == np.inf) and np.all(mx.numpy() == -np.inf)


def test_noalloc_refuses_what_exceeds_its_scratch():
    _C.init()
    # column route: 8 * C * inner bytes of partials > 1 MiB
    Cn, inner, outer = 70_000, 2, 64
    x = L.tensor(np.zeros(outer * Cn * inner, np.float32), device="hip")
    mn = L.Tensor.empty((Cn,), L.float32, "hip")
    mx = L.Tensor.empty((Cn,), L.float32, "hip")
    with pytest.raises(_C.ShapeMismatch):
        _C.call("lq_minmax_noalloc", x.data_ptr, outer, Cn, inner, mn.data_ptr, mx.data_ptr, None)
    # the allocating entry point takes it
    _C.call("lq_minmax", x.data_ptr, outer, Cn, inner, mn.data_ptr, mx.data_ptr, None)
    assert np.all(mn.numpy() == 0.0)


def test_noalloc_makes_no_pool_allocation():
    _C.init()
    x = L.tensor(np.ones(1 << 22, np.float32), device="hip")
    mn = L.Tensor.empty((1,), L.float32, "hip")
    mx = L.Tensor.empty((1,), L.float32, "hip")
    used0, res0 = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used0), C.byref(res0))
    _C.call("lq_minmax_noalloc", x.data_ptr, 1, 1, 1 << 22, mn.data_ptr, mx.data_ptr, None)
    used1, res1 = C.c_size_t(), C.c_size_t()
    _C.call("lq_memory_stats", C.byref(used1), C.byref(res1))
    assert (used1.value, res1.value) == (used0.value, res0.value)
    assert mn.numpy()[0] == 1.0 and mx.numpy()[0] == 1.0


def test_noalloc_takes_no_device_memory_at_all():
    """The pool's statistics do not see the library's own scratch (raw hipMalloc), so the contract
    is checked against the driver's free-memory figure, on a stream that has never been used: there
    lq_minmax has to allocate its 4 MiB workspace (which the figure shows), lq_minmax_noalloc
    nothing."""
    _C.init()
    x = L.tensor(np.arange(1 << 22, dtype=np.float32), device="hip")
    mn = L.Tensor.empty((1,), L.float32, "hip")
    mx = L.Tensor.empty((1,), L.float32, "hip")

    def free_bytes():
        _C.call("lq_sync", None)
        f, t = C.c_size_t(), C.c_size_t()
        _C.call("lq_device_memory_info", C.byref(f), C.byref(t))
        return f.value

    s1, s2 = C.c_void_p(), C.c_void_p()
    _C.call("lq_stream_create", C.byref(s1))
    _C.call("lq_stream_create", C.byref(s2))
    _C.call("lq_minmax_noalloc", x.data_ptr, 1, 1, 1 << 22, mn.data_ptr, mx.data_ptr, None)  # first use is behind us
    for s in (s1, s2):  # and so is whatever the runtime sets up at a stream's first launch
        _C.call("lq_fill_bytes", mn.data_ptr, 0, 4, s)
        _C.call("lq_sync", s)
    before = free_bytes()
    _C.call("lq_minmax_noalloc", x.data_ptr, 1, 1, 1 << 22, mn.data_ptr, mx.data_ptr, s1)
    _C.call("lq_sync", s1)
    assert free_bytes() == before
    assert mn.numpy()[0] == 0.0 and mx.numpy()[0] == float((1 << 22) - 1)
    # the allocating entry point on another fresh stream: the figure does see library scratch
    _C.call("lq_minmax", x.data_ptr, 1, 1, 1 << 22, mn.data_ptr, mx.data_ptr, s2)
    _C.call("lq_sync", s2)
    assert free_bytes() <= before - (4 << 20)
    assert mn.numpy()[0] == 0.0 and mx.numpy()[0] == float((1 << 22) - 1)
