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
