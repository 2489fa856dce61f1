"""In-band per-op profiler struct (mirror of python/athena/profiler.py:15-28)."""
import ctypes

from ._base import _LIB, check_call


class Profiler(ctypes.Structure):
    _fields_ = [("time", ctypes.c_float),              # ms
                ("input_memory", ctypes.c_float),      # MiB
                ("output_memory", ctypes.c_float),
                ("workspace_memory", ctypes.c_float)]


ProfilerHandle = ctypes.POINTER(Profiler)


def CreateProfiler():
    p = ProfilerHandle()
    check_call(_LIB.ProfilerAlloc(ctypes.byref(p)))
    return p.contents


def PrintProfiler(name, p):
    assert isinstance(p, Profiler)
    print('node=%-40s time=%-12f ms input_memory=%-4f MB output_memory=%-4f MB workspace_memory=%-4f MB'
          % (name, p.time, p.input_memory, p.output_memory, p.workspace_memory))
