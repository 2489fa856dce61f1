"""MI355X-native operator layer for Athena/TSplit: host-side mirror of the reference's
ctypes boundary over a from-scratch HIP (gfx950) implementation of libc_runtime_api.so."""
from . import gpu_links, gpu_memory_manager, ndarray, profiler, stream  # noqa: F401
from .ndarray import cpu, gpu  # noqa: F401
