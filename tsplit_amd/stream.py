"""Streams and events of the operator library: thin owners of the DLStream* / DLEvent* the C ABI
hands out.  Public names follow the reference's host module (python/athena/stream.py:10-54:
Stream, Event, create_stream_handle, create_event_handle, and the methods sync / query /
record), so code written against it runs unchanged."""
import ctypes

from ._base import _LIB, check_call


class _DeviceHandle(ctypes.Structure):
    """Layout shared by DLStream and DLEvent (src/common/dlarray.h:46-63): the device and a
    pointer to the runtime's own object."""
    _fields_ = [("device_id", ctypes.c_int), ("handle", ctypes.c_void_p)]


class DLStream(_DeviceHandle):
    pass


class DLEvent(_DeviceHandle):
    pass


DLStreamHandle = ctypes.POINTER(DLStream)
DLEventHandle = ctypes.POINTER(DLEvent)


class _Owned(object):
    """Owns one handle; releases it through `_destroy` when collected."""
    __slots__ = ["handle"]
    _destroy = None

    def __init__(self, handle):
        self.handle = handle

    def __del__(self):
        handle, self.handle = getattr(self, "handle", None), None
        if handle:
            getattr(_LIB, self._destroy)(handle)     # no check: the library may already be unloading


class Stream(_Owned):
    _destroy = "DLStreamDestroy"

    def sync(self):
        """Blocks until everything queued on the stream has finished."""
        check_call(_LIB.DLStreamSync(self.handle))


class Event(_Owned):
    _destroy = "DLEventDestroy"

    def record(self, stream):
        """Marks the current end of `stream` (None: the default stream)."""
        check_call(_LIB.DLEventRecord(stream.handle if stream else None, self.handle))

    def sync(self):
        check_call(_LIB.DLEventSync(self.handle))

    def query(self):
        """True once the recorded point has been reached."""
        return _LIB.DLEventQuery(self.handle) != 0


def _create(owner, pointer_type, maker, ctx):
    raw = pointer_type()
    check_call(getattr(_LIB, maker)(ctypes.c_size_t(ctx.device_id), ctypes.byref(raw)))
    return owner(raw)


def create_stream_handle(ctx):
    return _create(Stream, DLStreamHandle, "DLStreamCreate", ctx)


def create_event_handle(ctx):
    return _create(Event, DLEventHandle, "DLEventCreate", ctx)


# ---------------------------------------------------------------- recorded steps (HIP graphs)
class DLGraph(_DeviceHandle):
    pass


DLGraphHandle = ctypes.POINTER(DLGraph)


class _Keeper(object):
    """Device arrays born while a step was being recorded: the recorded kernels hold their
    addresses, so their memory goes back to the allocator only when the graph is gone."""
    __slots__ = ["handles", "rule", "open"]

    def __init__(self):
        self.handles, self.rule, self.open = [], 1, True

    def take(self, array_handle, rule):
        """Called by an array of this recording when it is collected; True if the keeper now
        owns the allocation."""
        if not self.open:
            return False
        self.handles.append(array_handle)
        self.rule = rule
        return True

    def release(self):
        self.open = False
        handles, self.handles = self.handles, []
        for h in handles:
            _LIB.DLArrayFree(h, ctypes.c_int(self.rule))


_recording_keeper = None          # the keeper of the recording in progress, if any


def current_keeper():
    return _recording_keeper


class Graph(_Owned):
    """A recorded step: `launch(stream)` replays every call recorded between the begin and the
    end of `recording(stream)`, with the arrays and scalars they had then."""
    __slots__ = ["_keeper"]
    _destroy = "TSplit_GraphDestroy"

    def __init__(self, handle, keeper):
        super().__init__(handle)
        self._keeper = keeper

    def launch(self, stream):
        check_call(_LIB.TSplit_GraphLaunch(self.handle, stream.handle))

    def __del__(self):
        super().__del__()
        keeper = getattr(self, "_keeper", None)
        if keeper is not None:
            keeper.release()


class recording(object):
    """with recording(stream) as rec: <issue one step on `stream`>  -> rec.graph

    Nothing issued inside the block runs; it is recorded.  Run the step once before (first-use
    set-up is refused while recording), keep host-visible calls (sync, asnumpy, copies without a
    stream) outside the block, and keep the arrays the step uses alive while the graph is in
    use; arrays created inside the block are kept alive by the graph itself."""

    def __init__(self, stream):
        self.stream, self.graph = stream, None

    def __enter__(self):
        global _recording_keeper
        if _recording_keeper is not None:
            raise RuntimeError("a step is already being recorded")
        check_call(_LIB.TSplit_StreamBeginRecord(self.stream.handle))
        _recording_keeper = self._keeper = _Keeper()
        return self

    def __exit__(self, exc_type, exc, tb):
        global _recording_keeper
        _recording_keeper = None
        raw = DLGraphHandle()
        ret = _LIB.TSplit_StreamEndRecord(self.stream.handle, ctypes.byref(raw))
        if ret != 0 or exc_type is not None:
            if ret == 0:
                _LIB.TSplit_GraphDestroy(raw)
            self._keeper.release()
            if exc_type is None:
                raise RuntimeError("the recording was invalidated by a call that cannot be recorded")
            return False
        self.graph = Graph(raw, self._keeper)
        return False
