"""What the device pool holds, for executors that poll it.  Function names follow the reference's
host module (python/athena/gpu_memory_manager.py:5-40)."""
import collections
import ctypes

from ._base import _LIB

PoolState = collections.namedtuple("PoolState", "used unused_unavailable unused_available")
_MIB = float(1 << 20)


def pool_state():
    """Bytes in use, bytes attached to used chunks as slack, bytes free for new tensors."""
    counters = (ctypes.c_size_t * 3)()
    _LIB.DLMemoryManager_GPU_Usage(*(ctypes.byref(counters, i * ctypes.sizeof(ctypes.c_size_t)) for i in range(3)))
    return PoolState(*(int(v) for v in counters))


def get_gpu_memory():
    """The same three figures keyed as the reference keys them, each with a `.value`."""
    st = pool_state()
    return {"used_size": ctypes.c_size_t(st.used), "unused_unavailable_size": ctypes.c_size_t(st.unused_unavailable),
            "unused_available_size": ctypes.c_size_t(st.unused_available)}


def print_gpu_memory():
    st = pool_state()
    print("Used: {} MB Unused available: {} MB".format(st.used / _MIB, st.unused_available / _MIB))


def print_gpu_used_memory(phase=None):
    print("Phase: {} Used: {} MB".format(phase, pool_state().used / _MIB))


def _pool_query(symbol, *args):
    answer = ctypes.c_int(0)
    getattr(_LIB, symbol)(*args, ctypes.byref(answer))
    return answer.value


def judge_malloc(shape):
    """1 if a float32 tensor of `shape` could be allocated from the pool now."""
    nbytes = 4
    for extent in shape:
        nbytes *= int(extent)
    return _pool_query("DLMemoryManager_Try_to_Malloc", ctypes.c_size_t(nbytes))


def _print_state(verbose):
    answer = ctypes.c_int(0)
    _LIB.DLMemoryManager_PrintState(ctypes.byref(answer), ctypes.c_int(verbose))
    return answer.value


def print_usage():
    """Prints the pool's chunk list; returns the number of free chunks."""
    return _print_state(1)


def judge_usage():
    """Number of free chunks in the pool."""
    return _print_state(0)
