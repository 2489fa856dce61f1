"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header
declares, has the reference's struct layouts, and its device-free runtime entry points
(host arrays, micro-tensor views, overlapped allocation, pool core) behave as specified.
No compute kernels are called here."""
import ctypes
import os
import re

import numpy as np
import pytest

from oracle import ops as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    txt = open(os.path.join(ROOT, "include", "c_runtime_api.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"^(?:int|void)\s+(\w+)\s*\(", txt, flags=re.M)))


def test_library_exports_every_declared_symbol():
    from tsplit_amd._base import _LIB
    syms = _declared_symbols()
    assert len(syms) >= 55
    missing = [s for s in syms if not hasattr(_LIB, s)]
    assert not missing, missing


def test_struct_layouts_match_reference():
    from tsplit_amd import ndarray, profiler, stream
    assert ctypes.sizeof(ndarray.DLContext) == 8
    assert ctypes.sizeof(ndarray.DLArray) == 32
    assert ndarray.DLArray.data.offset == 0 and ndarray.DLArray.ctx.offset == 8
    assert ndarray.DLArray.ndim.offset == 16 and ndarray.DLArray.shape.offset == 24
    assert ctypes.sizeof(stream.DLStream) == 16 and ctypes.sizeof(stream.DLEvent) == 16
    assert ctypes.sizeof(profiler.Profiler) == 16


def test_profiler_alloc_defaults():
    from tsplit_amd import profiler
    p = profiler.CreateProfiler()
    assert (p.time, p.input_memory, p.output_memory, p.workspace_memory) == (-1, -1, -1, -1)


def test_host_array_roundtrip_and_views(rng):
    from tsplit_amd import ndarray
    x = rng.normal(size=(10, 3, 2, 2)).astype(np.float32)
    a = ndarray.array(x, ndarray.cpu(0))
    assert a.shape == x.shape
    np.testing.assert_array_equal(a.asnumpy(), x)
    # uneven batch split 10 -> 3,3,2,2: zero-copy views that tile the parent bit-exactly
    a.split_tensor(4, "batch")
    assert [t.shape for t in a.sTensor] == O.split_shape(x.shape, 4) == [tuple(s) for s in ndarray.split_shape(x.shape, 4)]
    base = a.data_ptr
    for i, t in enumerate(a.sTensor):
        off, shp = O.micro_tensor_view(x.shape, 4, i)
        assert t.data_ptr == base + 4 * off and t.shape == shp
        np.testing.assert_array_equal(t.asnumpy(), x.ravel()[off:off + int(np.prod(shp))].reshape(shp))
    np.testing.assert_array_equal(np.concatenate([t.asnumpy() for t in a.sTensor]), x)
    # writing through a view lands in the parent
    a.sTensor[2][:] = np.full(a.sTensor[2].shape, 7, np.float32)
    assert (a.asnumpy()[6:8] == 7).all() and (a.asnumpy()[:6] == x[:6]).all()
    # "channel" view of an N == 1 tensor is a true channel slice
    y = rng.normal(size=(1, 6, 2, 2)).astype(np.float32)
    b = ndarray.array(y, ndarray.cpu(0))
    v = ndarray.slice_for_micro_tensor(b, 2, 4, "channel")
    off, shp = O.micro_tensor_view(y.shape, 4, 2, 1)
    assert v.shape == shp == (1, 1, 2, 2)
    np.testing.assert_array_equal(v.asnumpy(), y[:, 4:5])


def test_reuse_alloc_layout():
    from tsplit_amd import ndarray
    inp, out = ndarray.tensor_reuse((16,), (8,), 4, 1, ctx=ndarray.cpu(0))
    total, in_off, out_off = O.reuse_alloc_layout((16,), (8,), 4, 1)
    assert inp.data_ptr - out.data_ptr == in_off - out_off == 16
    assert inp.shape == (16,) and out.shape == (8,)
    # the overlap is real memory: the tail of `out` is the head of `inp`
    out[:] = np.arange(8, dtype=np.float32)
    assert list(inp.asnumpy()[:4]) == [4, 5, 6, 7]


def test_copy_size_mismatch_is_an_error():
    from tsplit_amd import ndarray
    from tsplit_amd._base import _LIB
    a = ndarray.empty((4,), ndarray.cpu(0))
    b = ndarray.empty((5,), ndarray.cpu(0))
    assert _LIB.DLArrayCopyFromTo(a.handle, b.handle, None) == -1


# ---------------------------------------------------------------- pool core (fake device)
@pytest.fixture
def pool_lib():
    path = os.path.join(ROOT, "tsplit_amd", "lib", "libtsplit_pool_host.so")
    lib = ctypes.CDLL(path)
    lib.pool_test_create.restype = ctypes.c_void_p
    lib.pool_test_create.argtypes = [ctypes.c_size_t] * 3
    lib.pool_test_malloc.restype = ctypes.c_size_t
    lib.pool_test_malloc.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.pool_test_free.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.pool_test_try.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    lib.pool_test_usage.argtypes = [ctypes.c_void_p] + [ctypes.POINTER(ctypes.c_size_t)] * 3
    lib.pool_test_free_chunks.argtypes = [ctypes.c_void_p]
    lib.pool_test_reserved.restype = ctypes.c_size_t
    lib.pool_test_reserved.argtypes = [ctypes.c_void_p]
    lib.pool_test_backing_calls.argtypes = [ctypes.c_void_p]
    lib.pool_test_destroy.argtypes = [ctypes.c_void_p]
    return lib


def _usage(lib, h):
    u = [ctypes.c_size_t(0) for _ in range(3)]
    lib.pool_test_usage(h, *[ctypes.byref(x) for x in u])
    return tuple(x.value for x in u)


def test_pool_best_fit_split_coalesce(pool_lib):
    MiB = 1 << 20
    h = pool_lib.pool_test_create(1024 * MiB, 64 * MiB, 1 << 62)
    a = pool_lib.pool_test_malloc(h, 1000)          # rounds to 1024, splits the 64 MiB slab
    b = pool_lib.pool_test_malloc(h, 10 * MiB)
    c = pool_lib.pool_test_malloc(h, 300)
    assert a and b and c and a % 256 == 0 and b % 256 == 0
    assert b == a + 1024 and c == b + 10 * MiB      # carved front to back
    assert pool_lib.pool_test_backing_calls(h) == 1 and pool_lib.pool_test_reserved(h) == 64 * MiB
    used, uu, ua = _usage(pool_lib, h)
    assert used == 1000 + 10 * MiB + 300 and uu == 24 + 212
    assert ua == 1024 * MiB - used - uu             # free chunk + what the device could still give
    # free the middle block: one more free chunk; then its neighbours: everything coalesces
    assert pool_lib.pool_test_free(h, b) == 1
    assert pool_lib.pool_test_free_chunks(h) == 2
    # best fit: a 5 MiB request goes into the 10 MiB hole, not the big tail
    d = pool_lib.pool_test_malloc(h, 5 * MiB)
    assert d == b
    assert pool_lib.pool_test_free(h, d) == 1
    assert pool_lib.pool_test_free(h, a) == 1 and pool_lib.pool_test_free(h, c) == 1
    assert pool_lib.pool_test_free_chunks(h) == 1   # fully coalesced
    assert _usage(pool_lib, h)[0] == 0
    assert pool_lib.pool_test_free(h, a) == 0       # double free is reported, not fatal
    pool_lib.pool_test_destroy(h)


def test_pool_split_rule_and_growth_and_limit(pool_lib):
    MiB = 1 << 20
    h = pool_lib.pool_test_create(1024 * MiB, 64 * MiB, 200 * MiB)
    a = pool_lib.pool_test_malloc(h, 40 * MiB)      # 64 MiB slab: 64 <= 2*40 and slack < 128 MiB => no split
    used, uu, ua = _usage(pool_lib, h)
    assert used == 40 * MiB and uu == 24 * MiB
    b = pool_lib.pool_test_malloc(h, 100 * MiB)     # larger than a slab: dedicated slab of exactly that size
    assert b and pool_lib.pool_test_backing_calls(h) == 2 and pool_lib.pool_test_reserved(h) == 164 * MiB
    assert pool_lib.pool_test_try(h, 36 * MiB) == 1 and pool_lib.pool_test_try(h, 37 * MiB) == 0   # limit 200 MiB
    assert pool_lib.pool_test_malloc(h, 37 * MiB) == 0                                               # OOM -> NULL
    assert pool_lib.pool_test_free(h, b) == 1
    assert pool_lib.pool_test_try(h, 100 * MiB) == 1                                                 # from the freed slab
    pool_lib.pool_test_destroy(h)


def test_header_compiles_as_c_and_cxx_and_links(tmp_path):
    """A C translation unit and a C++ one that include the public header, take the address of a few
    entry points with their declared types, and link against the built library: the header is
    self-contained plain C, and the declarations agree with the definitions' C linkage."""
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib_dir = os.path.join(root, "tsplit_amd", "lib")
    if not os.path.exists(os.path.join(lib_dir, "libc_runtime_api.so")):
        pytest.skip("library not built")
    body = '''
#include "c_runtime_api.h"
#include <stddef.h>
typedef int (*relu_fn)(const DLArrayHandle, DLArrayHandle, DLStreamHandle, ProfilerHandle);
typedef int (*conv_fn)(const DLArrayHandle, const DLArrayHandle, DLArrayHandle, const int, const int, const int,
                       DLStreamHandle, ProfilerHandle);
int main(void) {
  relu_fn r = DLGpuRelu;
  conv_fn c = CuDNN_DLGpuConv2d;
  DLArray a;
  a.data = NULL;
  a.ndim = 0;
  a.shape = NULL;
  return (r != NULL && c != NULL && a.data == NULL && a.ndim == 0 && a.shape == NULL && sizeof(DLArray) == 32 && sizeof(DLContext) == 8 && sizeof(Profiler) == 16) ? 0 : 1;
}
'''
    for compiler, name, std in (("gcc", "t.c", "-std=c99"), ("g++", "t.cpp", "-std=c++11")):
        if shutil.which(compiler) is None:
            pytest.skip(compiler + " not found")
        src = tmp_path / name
        src.write_text(body)
        exe = tmp_path / (name + ".out")
        cmd = [compiler, std, "-Wall", "-Werror", "-I", os.path.join(root, "include"), str(src), "-o", str(exe),
               "-L", lib_dir, "-lc_runtime_api", "-Wl,-rpath," + lib_dir, "-Wl,--allow-shlib-undefined"]
        done = subprocess.run(cmd, capture_output=True, text=True)
        assert done.returncode == 0, done.stderr
        ran = subprocess.run([str(exe)], capture_output=True, text=True)
        assert ran.returncode == 0, ran.stderr
