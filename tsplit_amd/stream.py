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
