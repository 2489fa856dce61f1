"""Pool introspection (mirror of python/athena/gpu_memory_manager.py:5-40)."""
import ctypes

from ._base import _LIB


def get_gpu_memory():
    usage = {k: ctypes.c_size_t(0) for k in ("used_size", "unused_unavailable_size", "unused_available_size")}
    _LIB.DLMemoryManager_GPU_Usage(ctypes.byref(usage["used_size"]),
                                   ctypes.byref(usage["unused_unavailable_size"]),
                                   ctypes.byref(usage["unused_available_size"]))
    return usage


def print_gpu_memory():
    u = get_gpu_memory()
    print("Used: {} MB Unused available: {} MB".format(u["used_size"].value / 2 ** 20,
                                                       u["unused_available_size"].value / 2 ** 20))


def judge_malloc(shape):
    """1 if a float32 tensor of `shape` could be allocated from the pool now."""
    num = 1
    for i in shape:
        num *= i
    t = ctypes.c_int(0)
    _LIB.DLMemoryManager_Try_to_Malloc(ctypes.c_size_t(num * 4), ctypes.byref(t))
    return t.value


def print_usage():
    t = ctypes.c_int(0)
    _LIB.DLMemoryManager_PrintState(ctypes.byref(t), ctypes.c_int(1))
    return t.value


def judge_usage():
    """Number of free chunks in the pool."""
    t = ctypes.c_int(0)
    _LIB.DLMemoryManager_PrintState(ctypes.byref(t), ctypes.c_int(0))
    return t.value
