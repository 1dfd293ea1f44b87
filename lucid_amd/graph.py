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


_captures_open = 0


def is_capturing() -> bool:
    """True inside a ``capture()`` block of this module (what is launched now will be replayed)."""
    return _captures_open > 0


@contextlib.contextmanager
def capture():
    global _captures_open
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
    _captures_open += 1
    try:
        yield g
        ok = True
    finally:
        _captures_open -= 1
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
    """A forward captured once per contiguous slice of the batch, the slices as parallel branches of
    ONE graph (each captured on a stream of its own, forked from and joined to the capture stream
    by events).  A chain of short dependent kernels leaves most of the chip idle while each kernel
    ramps up and drains; independent slices of the batch fill those gaps for one another.

    Only for forwards whose result for a row does not depend on the other rows of the batch
    (static quantization; NOT dynamic per-tensor quantization, whose ranges are taken over the
    whole batch).  ``output`` holds the slices' results, concatenated along axis 0."""

    def __init__(self) -> None:
        self.graph: Graph | None = None
        self.branches = 0
        self.output = None
        self._events: list = []
        self._streams: list = []

    def replay(self) -> None:
        if self.graph is None:
            raise _C.LucidError("graph was not captured")
        self.graph.replay()

    def destroy(self) -> None:
        if self.graph is not None:
            self.graph.destroy()
            self.graph = None
        for ev in self._events:
            _C.call("lq_event_destroy", ev)
        for st in self._streams:
            _C.call("lq_stream_destroy", st)
        self._events, self._streams = [], []

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


def capture_split(fn, x, parts: int = 2) -> SplitGraph:
    """Capture ``fn`` on ``parts`` contiguous slices of ``x`` along axis 0 as parallel branches of one
    graph (see ``SplitGraph``).  ``fn(x_slice)`` returns one device tensor whose axis 0 is the
    slice's batch.  Run ``fn`` on each slice size once before capturing (host-side scalars, kernel
    tuning)."""
    from ._tensor import Tensor

    batch = x.shape[0]
    parts = max(1, min(int(parts), batch))
    bounds = [batch * i // parts for i in range(parts + 1)]
    sg = SplitGraph()
    sg.branches = parts

    def new_event():
        ev = C.c_void_p()
        _C.call("lq_event_create", C.byref(ev))
        sg._events.append(ev)
        return ev

    try:
        fork = new_event()
        for _ in range(parts - 1):
            st = C.c_void_p()
            _C.call("lq_stream_create", C.byref(st))
            sg._streams.append(st)
        with capture() as g:
            main = _C.current_stream()
            _C.call("lq_event_record", fork, main)
            joins = []
            try:
                for i, (lo, hi) in enumerate(zip(bounds[:-1], bounds[1:])):
                    st = main if i == 0 else sg._streams[i - 1]
                    if i:
                        _C.call("lq_stream_wait_event", st, fork)  # the stream joins the capture here
                    _C.set_current_stream(st)
                    y = fn(x.row_range(lo, hi))
                    if sg.output is None:
                        # allocated during the capture, so it stays pinned like the other captured tensors
                        sg.output = Tensor.empty((batch, *y.shape[1:]), y.dtype, "hip")
                    dst = sg.output.row_range(lo, hi)
                    _C.call("lq_d2d", dst.data_ptr, y.data_ptr, y.nbytes, st)
                    if i:
                        join = new_event()
                        _C.call("lq_event_record", join, st)
                        joins.append(join)
            finally:
                _C.set_current_stream(main)
            for join in joins:
                _C.call("lq_stream_wait_event", main, join)
        sg.graph = g
    except Exception:
        sg.destroy()
        raise
    return sg
