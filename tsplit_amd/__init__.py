"""MI355X-native operator layer for Athena/TSplit: host-side mirror of the reference's
ctypes boundary over a from-scratch HIP (gfx950) implementation of libc_runtime_api.so.

Submodules load on first use, so that `python -m tsplit_amd.build` can run before the
library exists; everything else needs the built library and raises if it is missing."""
import importlib

_SUBMODULES = ("gpu_links", "gpu_memory_manager", "ndarray", "profiler", "stream", "trainer", "build")


def __getattr__(name):
    if name in _SUBMODULES:
        return importlib.import_module("." + name, __name__)
    if name in ("cpu", "gpu"):
        return getattr(importlib.import_module(".ndarray", __name__), name)
    raise AttributeError(name)
