"""Loads the C-ABI operator library and holds the small ctypes helpers.

Mirror of the reference's python/athena/_base.py:62-91 (one global CDLL, `check_call`,
`c_array`).  The library must have been built (python -m tsplit_amd.build); there is no
fallback: a missing library raises at import, as the reference's import does.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TSPLIT_LIB_PATH overrides the in-tree location (e.g. to try another build of the library)
LIB_PATH = os.environ.get("TSPLIT_LIB_PATH") or os.path.join(_HERE, "lib", "libc_runtime_api.so")


def _load_lib():
    if not os.path.exists(LIB_PATH):
        raise OSError(
            f"{LIB_PATH} is missing: build it with `python -m tsplit_amd.build` "
            "(hipcc, gfx950). There is no CPU fallback for the operator library.")
    lib = ctypes.CDLL(LIB_PATH, ctypes.RTLD_GLOBAL)
    lib.DLMemoryManager_PrintState.restype = None
    lib.DLMemoryManager_Try_to_Malloc.restype = None
    lib.DLMemoryManager_GPU_Usage.restype = None
    for name in ("cudnn_init", "cublas_init", "cusp_init", "cuda_init"):
        getattr(lib, name).restype = None
    return lib


_LIB = _load_lib()


def check_call(ret):
    """Every runtime entry point returns 0 on success."""
    if ret != 0:
        raise RuntimeError(f"libc_runtime_api call failed with code {ret}")


def c_array(ctype, values):
    return (ctype * len(values))(*values)


def get_array_memory(shape):
    """Size of a float32 tensor in MiB."""
    n = 1.0
    for s in shape:
        n *= s
    return n * 4 / (2 ** 20)
