"""Host-side mirror of the reference's position / chunk loop and of a recorded
single-token step.

The reference's serving thread walks a request as: the prompt in chunks of
`sequence_chunk_size` positions, a shorter last chunk, then one position at a time
(src/serving/start copy.rs:71-113); every operator of the graph is run once per such
call.  `schedule_calls` returns those (position_index, position_interval) pairs;
`StepGraph` records the launches of one single-token step into a HIP graph so that the
per-token loop costs one launch instead of two per layer; `SideStream` lets the two
independent halves of a mixed step (a prompt chunk, one new token of the other
sequences) run side by side."""
import ctypes

from ._lib import check, load_library


class _Call(ctypes.Structure):
    _fields_ = [("position_index", ctypes.c_size_t), ("position_interval", ctypes.c_size_t)]


def schedule_calls(prompt_begin, prompt_end, chunk, generation_end):
    """[(position_index, position_interval), ...] for one request."""
    lib = load_library()
    n = ctypes.c_size_t(0)
    room = max(1, (max(prompt_end - prompt_begin, 0) + max(chunk, 1) - 1) // max(chunk, 1)
               + max(generation_end - prompt_end, 0))
    calls = (_Call * room)()
    check(lib.ellm_schedule_calls(prompt_begin, prompt_end, chunk, generation_end,
                                  ctypes.cast(calls, ctypes.c_void_p), room, ctypes.byref(n)))
    return [(calls[i].position_index, calls[i].position_interval) for i in range(n.value)]


def positions_advance(positions, by=1, stream=None):
    """positions (uint32/int32 device tensor) += by, in stream order."""
    from .attention import _stream_ptr

    check(load_library().ellm_positions_advance(ctypes.c_void_p(positions.data_ptr()),
                                                positions.numel(), by, _stream_ptr(stream)))


class SideStream:
    """A second stream of the library's (ellm_side_stream_*).  Pass the object as `stream=` to
    the operators whose launches may run beside those of the caller's stream:

        side.fork(stream); chunk_op.run(..., stream=stream); token_op.run_ragged(..., stream=side)
        side.join(stream)

    also between StepGraph's begin and end, where the side launches become a parallel branch."""

    def __init__(self):
        self._lib = load_library()
        self._handle = ctypes.c_void_p()
        check(self._lib.ellm_side_stream_create(ctypes.byref(self._handle)))

    @property
    def cuda_stream(self):
        return self._lib.ellm_side_stream_get(self._handle) or 0

    def fork(self, stream=None):
        from .attention import _stream_ptr

        check(self._lib.ellm_side_stream_fork(self._handle, _stream_ptr(stream)))

    def join(self, stream=None):
        from .attention import _stream_ptr

        check(self._lib.ellm_side_stream_join(self._handle, _stream_ptr(stream)))

    def close(self):
        if self._handle:
            check(self._lib.ellm_side_stream_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class StepGraph:
    """with StepGraph(stream) as g: <launches on `stream`> ; then g.launch() per step."""

    def __init__(self, stream):
        self._lib = load_library()
        self._stream = stream
        self._handle = ctypes.c_void_p()

    def __enter__(self):
        check(self._lib.ellm_graph_begin(ctypes.c_void_p(self._stream.cuda_stream)))
        return self

    def __exit__(self, exc_type, exc, tb):
        handle = ctypes.c_void_p()
        status = self._lib.ellm_graph_end(ctypes.c_void_p(self._stream.cuda_stream),
                                          ctypes.byref(handle))
        if exc_type is None:
            check(status)
            self._handle = handle
        elif status == 0:
            self._lib.ellm_graph_destroy(handle)
        return False

    def launch(self, stream=None):
        s = stream if stream is not None else self._stream
        check(self._lib.ellm_graph_launch(self._handle, ctypes.c_void_p(s.cuda_stream)))

    def close(self):
        if self._handle:
            check(self._lib.ellm_graph_destroy(self._handle))
            self._handle = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
