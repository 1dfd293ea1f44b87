"""HIP-graph capture of a fixed-shape forward pass.

A quantized network's forward is a chain of short kernels; driven from Python
the GPU waits on the interpreter.  ``capture()`` records everything launched
inside the ``with`` block into a HIP graph that ``replay()`` re-issues with a
single launch.  The tensors created during capture (inputs excepted) keep
their device memory for the lifetime of the graph, so replays read the same
input buffer and write the same output buffer:

    y = model(x)                      # eager warm-up: caches host-side scalars
    with lucid_amd.graph.capture() as g:
        y = model(x)
    x.copy_from(new_batch); g.replay(); result = y.numpy()

Nothing that talks to the host may run during capture (``.item()``,
``.numpy()``, uploads).
"""

from __future__ import annotations

import contextlib
import ctypes as C

from . import _C


class Graph:
    def __init__(self) -> None:
        self.id = None
        self._stream = None

    def replay(self) -> None:
        """Launch the captured work on the current stream."""
        if self.id is None:
            raise _C.LucidError("graph was not captured")
        _C.call("lq_graph_launch", self.id, None)

    def destroy(self) -> None:
        if self.id is not None:
            _C.call("lq_graph_destroy", self.id)
            self.id = None
        if self._stream is not None:
            _C.call("lq_stream_destroy", self._stream)
            self._stream = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


@contextlib.contextmanager
def capture():
    _C.init()
    g = Graph()
    stream = C.c_void_p()
    _C.call("lq_stream_create", C.byref(stream))
    g._stream = stream
    _C.call("lq_sync", None)  # everything issued so far is done before capture starts
    gid = C.c_int()
    prev = _C.current_stream()
    _C.call("lq_graph_begin", stream, C.byref(gid))
    _C.set_current_stream(stream)
    ok = False
    try:
        yield g
        ok = True
    finally:
        _C.set_current_stream(prev)
        try:
            _C.call("lq_graph_end", stream, gid.value)
            g.id = gid.value
        except Exception:
            # the capture was invalidated (or its body raised and left it unusable): drop the
            # id so that the blocks allocated during the capture are unpinned
            _C.load().lq_graph_destroy(gid.value)
            g.destroy()
            if ok:
                raise
        if not ok:
            # the body raised: whatever was captured is not a usable graph
            if g.id is None:
                _C.load().lq_graph_destroy(gid.value)
            g.destroy()


class SplitGraph:
    """A forward captured once per contiguous slice of the batch, each slice on a stream of its own,
    replayed together.  A chain of short dependent kernels leaves most of the chip idle while each
    kernel ramps up and drains; independent slices of the batch fill those gaps for one another.

    Only for forwards whose result for a row does not depend on the other rows of the batch
    (static quantization; NOT dynamic per-tensor quantization, whose ranges are taken over the
    whole batch).  ``output`` holds the slices' results, concatenated along axis 0."""

    def __init__(self) -> None:
        self.graphs: list[Graph] = []
        self.output = None
        self._fork = None
        self._joins: list = []
        self._streams: list = []  # replay streams: non-blocking, so the slices overlap even next to the default stream

    def replay(self) -> None:
        """Launch every slice's graph on its own stream; work queued on the current stream
        afterwards waits for all of them."""
        cur = _C.current_stream()
        _C.call("lq_event_record", self._fork, cur)
        # every slice is launched before the current stream is touched again: when that is the
        # default stream, each operation on it orders all the other streams' later work behind it
        for g, st, ev in zip(self.graphs, self._streams, self._joins):
            _C.call("lq_stream_wait_event", st, self._fork)
            _C.call("lq_graph_launch", g.id, st)
            _C.call("lq_event_record", ev, st)
        for ev in self._joins:
            _C.call("lq_stream_wait_event", cur, ev)

    def destroy(self) -> None:
        for g in self.graphs:
            g.destroy()
        self.graphs = []
        for ev in [self._fork, *self._joins]:
            if ev is not None:
                _C.call("lq_event_destroy", ev)
        self._fork, self._joins = None, []
        for st in self._streams:
            _C.call("lq_stream_destroy", st)
        self._streams = []

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def capture_split(fn, x, parts: int = 2) -> SplitGraph:
    """Capture ``fn`` on ``parts`` contiguous slices of ``x`` along axis 0 (see ``SplitGraph``).
    ``fn(x_slice)`` returns one device tensor whose axis 0 is the slice's batch.  Run ``fn`` on
    each slice size once before capturing (host-side scalars, kernel tuning)."""
    from ._tensor import Tensor

    batch = x.shape[0]
    parts = max(1, min(int(parts), batch))
    bounds = [batch * i // parts for i in range(parts + 1)]
    sg = SplitGraph()
    ev = C.c_void_p()
    _C.call("lq_event_create", C.byref(ev))
    sg._fork = ev
    try:
        for lo, hi in zip(bounds[:-1], bounds[1:]):
            xs = x.row_range(lo, hi)
            with capture() as g:
                y = fn(xs)
                if sg.output is None:
                    # allocated during the first capture, so it stays pinned like the other captured tensors
                    sg.output = Tensor.empty((batch, *y.shape[1:]), y.dtype, "hip")
                dst = sg.output.row_range(lo, hi)
                _C.call("lq_d2d", dst.data_ptr, y.data_ptr, y.nbytes, _C.current_stream())
            sg.graphs.append(g)
            j = C.c_void_p()
            _C.call("lq_event_create", C.byref(j))
            sg._joins.append(j)
            st = C.c_void_p()
            _C.call("lq_stream_create_nonblocking", C.byref(st))
            sg._streams.append(st)
    except Exception:
        sg.destroy()
        raise
    return sg
