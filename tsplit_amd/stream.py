"""Stream and event wrappers over DLStream*/DLEvent* (mirror of python/athena/stream.py:10-54)."""
import ctypes

from ._base import _LIB, check_call


class DLStream(ctypes.Structure):
    _fields_ = [("device_id", ctypes.c_int), ("handle", ctypes.c_void_p)]


DLStreamHandle = ctypes.POINTER(DLStream)


class Stream(object):
    __slots__ = ["handle"]

    def __init__(self, handle):
        self.handle = handle

    def __del__(self):
        if self.handle:
            _LIB.DLStreamDestroy(self.handle)
            self.handle = None

    def sync(self):
        check_call(_LIB.DLStreamSync(self.handle))


def create_stream_handle(ctx):
    handle = DLStreamHandle()
    check_call(_LIB.DLStreamCreate(ctypes.c_size_t(ctx.device_id), ctypes.byref(handle)))
    return Stream(handle)


class DLEvent(ctypes.Structure):
    _fields_ = [("device_id", ctypes.c_int), ("handle", ctypes.c_void_p)]


DLEventHandle = ctypes.POINTER(DLEvent)


class Event(object):
    __slots__ = ["handle"]

    def __init__(self, handle):
        self.handle = handle

    def __del__(self):
        if self.handle:
            _LIB.DLEventDestroy(self.handle)
            self.handle = None

    def sync(self):
        check_call(_LIB.DLEventSync(self.handle))

    def query(self):
        return bool(_LIB.DLEventQuery(self.handle))

    def record(self, stream):
        check_call(_LIB.DLEventRecord(stream.handle if stream else None, self.handle))


def create_event_handle(ctx):
    handle = DLEventHandle()
    check_call(_LIB.DLEventCreate(ctypes.c_size_t(ctx.device_id), ctypes.byref(handle)))
    return Event(handle)
