"""NDArray container over the DLArray C struct.

Host-side mirror of the reference's python/athena/ndarray.py (same names and call
sequences: `array`, `empty`, `NDArray.asnumpy/_sync_copyfrom/copyto/split_tensor/
delete_itself/malloc_itself`, `tensor_reuse`, `slice_for_micro_tensor`, `split_shape`),
written for Python 3.  Differences from the reference, all on the host side:
  * the three per-array events (ndarray.py:94-97) are created on first use, not per array;
  * micro-tensor views keep their parent alive and release their own struct when
    collected (the reference leaks them).
"""
import ctypes

import numpy as np

from ._base import _LIB, c_array, check_call
from .stream import create_event_handle, current_keeper

# 0: raw device malloc/free per tensor; != 0: pooled allocator (ndarray.py:8)
MEMORY_MANAGE_RULE = 1


class DLContext(ctypes.Structure):
    _fields_ = [("device_id", ctypes.c_int), ("device_type", ctypes.c_int)]
    MASK2STR = {1: "cpu", 2: "gpu"}

    def __init__(self, device_id=0, device_type=1):
        super().__init__()
        self.device_id = device_id
        self.device_type = device_type

    def __repr__(self):
        return "%s(%d)" % (DLContext.MASK2STR[self.device_type], self.device_id)


class DLArray(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p),
                ("ctx", DLContext),
                ("ndim", ctypes.c_int),
                ("shape", ctypes.POINTER(ctypes.c_int64))]


DLArrayHandle = ctypes.POINTER(DLArray)


def cpu(dev_id=0):
    return DLContext(dev_id, 1)


def gpu(dev_id=0):
    return DLContext(dev_id, 2)


def is_gpu_ctx(ctx):
    return bool(ctx) and ctx.device_type == 2


class NDArray(object):
    """A buffer object: no arithmetic, only allocation, copies and micro-tensor views."""
    __slots__ = ["handle", "auto_deleted", "swap", "in_gpu", "_events", "splitted", "sTensor",
                 "split_number", "split_dimension", "_owner", "_is_view", "_keeper"]

    def __init__(self, handle, auto_deleted=True, owner=None, is_view=False):
        self.handle = handle
        self.auto_deleted = auto_deleted
        self.splitted = False
        self.sTensor = []
        self.split_number = 1
        self.split_dimension = None
        self.swap = False
        self.in_gpu = True
        self._events = {}
        self._owner = owner          # keeps the parent allocation alive for views
        self._is_view = is_view
        self._keeper = current_keeper()     # set while a step is being recorded into a graph

    def __del__(self):
        h = getattr(self, "handle", None)
        if not h:
            return
        if self._is_view:
            # a view owns its struct and shape but not its data
            h.contents.data = None
            _LIB.DLArrayFree(h, ctypes.c_int(MEMORY_MANAGE_RULE))
        elif self.auto_deleted:
            # an array born inside a recorded step outlives this object: the graph replays into it
            keeper = getattr(self, "_keeper", None)
            if keeper is None or h.contents.ctx.device_type != 2 or not keeper.take(h, MEMORY_MANAGE_RULE):
                _LIB.DLArrayFree(h, ctypes.c_int(MEMORY_MANAGE_RULE))
        self.handle = None

    # ---- events used by swapping executors (created lazily) ----
    def _event(self, name):
        ev = self._events.get(name)
        if ev is None:
            ev = self._events[name] = create_event_handle(self.ctx)
        return ev

    cpu2gpu_event = property(lambda self: self._event("cpu2gpu"))
    gpu_event = property(lambda self: self._event("gpu"))
    gpu2cpu_event = property(lambda self: self._event("gpu2cpu"))

    def is_swapout_ok(self):
        return self.gpu2cpu_event.query()

    def is_swapin_ok(self):
        if self.cpu2gpu_event.query():
            self.in_gpu = True
            return 1
        return 0

    # ---- micro-tensor split ----
    def split_tensor(self, total_number, dimension="batch"):
        """Populate self.sTensor with `total_number` zero-copy views."""
        if self.split_number == total_number and self.split_dimension == dimension and self.sTensor:
            return
        self.splitted = True
        self.split_number = total_number
        self.split_dimension = dimension
        self.sTensor = [slice_for_micro_tensor(self, i, total_number, dimension) for i in range(total_number)]

    def merge(self):
        self.splitted = False
        self.in_gpu = True
        # the views refer to this array and this array lists them: dropping the list breaks that cycle, so
        # the array is freed when its last outside reference goes and not when the collector next runs
        self.sTensor = []

    # ---- drop / re-acquire the data pointer, keeping the struct ----
    def delete_itself(self):
        if self.in_gpu:
            self.in_gpu = False
            check_call(_LIB.DLArrayFreeSelf(self.handle, ctypes.c_int(MEMORY_MANAGE_RULE)))

    def malloc_itself(self):
        check_call(_LIB.DLArrayAllocSelf(self.handle, ctypes.c_int(MEMORY_MANAGE_RULE)))
        self.in_gpu = True

    @property
    def shape(self):
        c = self.handle.contents
        return tuple(c.shape[i] for i in range(c.ndim))

    @property
    def ctx(self):
        return self.handle.contents.ctx

    @property
    def data_ptr(self):
        return self.handle.contents.data

    def __setitem__(self, in_slice, value):
        if not isinstance(in_slice, slice) or in_slice.start is not None or in_slice.stop is not None:
            raise ValueError("Array only support set from numpy array")
        if isinstance(value, NDArray):
            if value.handle is not self.handle:
                value.copyto(self)
        elif isinstance(value, (np.ndarray, np.generic)):
            self._sync_copyfrom(value)
        else:
            raise TypeError("type %s not supported" % str(type(value)))

    def _sync_copyfrom(self, source_array, data_type=np.float32):
        """Synchronous copy from a numpy array.  data_type np.int32 stores the 32-bit integers
        as they are (the index arrays of a sparse matrix, python/athena/ndarray.py:198-219)."""
        source_array = np.ascontiguousarray(source_array, dtype=data_type)
        if source_array.shape != self.shape:
            raise ValueError("array shape do not match the shape of NDArray")
        if source_array.dtype == np.int32:
            source_array = source_array.view(np.float32)
        elif source_array.dtype != np.float32:
            raise TypeError("only float32 and int32 elements are stored, not %s" % source_array.dtype)
        src, shape = NDArray._numpyasarray(source_array)
        check_call(_LIB.DLArrayCopyFromTo(ctypes.byref(src), self.handle, None))
        _ = shape

    def _async_copyfrom(self, source_array, stream, event=None):
        check_call(_LIB.DLArrayCopyFromTo(source_array.handle, self.handle, stream.handle))
        if event is not None:
            event.record(stream)

    def async_h2d(self, source_array, stream_handle, event_handle=None):
        assert self.ctx.device_type == 2 and source_array.ctx.device_type == 1 and stream_handle
        self._async_copyfrom(source_array, stream_handle, event_handle)

    def async_d2h(self, source_array, stream_handle, event_handle=None):
        assert self.ctx.device_type == 1 and source_array.ctx.device_type == 2 and stream_handle
        self._async_copyfrom(source_array, stream_handle, event_handle)

    def to_swap(self):
        self.swap = True

    @staticmethod
    def _numpyasarray(np_data):
        assert np_data.flags["C_CONTIGUOUS"] and np_data.dtype == np.float32
        arr = DLArray()
        shape = c_array(ctypes.c_int64, np_data.shape)
        arr.data = np_data.ctypes.data_as(ctypes.c_void_p)
        arr.shape = shape
        arr.ndim = np_data.ndim
        arr.ctx = cpu(0)
        return arr, shape

    def asnumpy(self):
        out = np.empty(self.shape, dtype=np.float32)
        arr, shape = NDArray._numpyasarray(out)
        check_call(_LIB.DLArrayCopyFromTo(self.handle, ctypes.byref(arr), None))
        _ = shape
        return out

    def copyto(self, target, stream_handle=None):
        if isinstance(target, DLContext):
            target = empty(self.shape, target)
        if not isinstance(target, NDArray):
            raise ValueError("Unsupported target type %s" % str(type(target)))
        check_call(_LIB.DLArrayCopyFromTo(self.handle, target.handle,
                                          stream_handle.handle if stream_handle else None))
        return target


def array(arr, ctx, stream_handle=None, event_handle=None):
    """New array on `ctx` holding a float32 copy of `arr` (synchronous copy)."""
    arr = np.asarray(arr)
    ret = empty(arr.shape, ctx)
    ret._sync_copyfrom(arr)
    return ret


def empty(shape, ctx=cpu(0)):
    cshape = c_array(ctypes.c_int64, tuple(int(s) for s in shape))
    handle = DLArrayHandle()
    check_call(_LIB.DLArrayAlloc(cshape, ctypes.c_int64(len(cshape)), ctx, ctypes.byref(handle),
                                 ctypes.c_int(MEMORY_MANAGE_RULE)))
    return NDArray(handle)


class ND_Sparse_Array(object):
    """CSR matrix on a device: values, row pointers and column indices as three 1-D arrays
    (python/athena/ndarray.py:412-425)."""
    __slots__ = ["data", "row", "col", "nrow", "ncol"]

    def __init__(self, data, row, col, nrow, ncol):
        self.data = data
        self.row = row
        self.col = col
        self.nrow = nrow
        self.ncol = ncol

    @property
    def shape(self):
        return (self.nrow, self.ncol)


def sparse_array(values, indices, shape, ctx=cpu(0)):
    """CSR copy on `ctx` of the matrix with `values` at `indices` = (rows, cols); entries
    with equal coordinates are summed and every row's columns come out ascending, as
    scipy.sparse.csr_matrix builds them (python/athena/ndarray.py:428-455)."""
    assert len(shape) == len(indices) == 2
    assert len(values) == len(indices[0]) == len(indices[1])
    rows = np.asarray(indices[0], dtype=np.int64)
    cols = np.asarray(indices[1], dtype=np.int64)
    vals = np.asarray(values, dtype=np.float32)
    assert rows.size == 0 or (rows.min() >= 0 and rows.max() < shape[0] and cols.min() >= 0 and cols.max() < shape[1])
    key = rows * int(shape[1]) + cols
    uniq, inverse = np.unique(key, return_inverse=True)
    summed = np.zeros(uniq.shape, dtype=np.float32)
    np.add.at(summed, inverse, vals)
    urows, ucols = uniq // int(shape[1]), uniq % int(shape[1])
    indptr = np.zeros(int(shape[0]) + 1, dtype=np.int32)
    np.cumsum(np.bincount(urows, minlength=int(shape[0])), out=indptr[1:])
    values_ret = empty(summed.shape, ctx)
    values_ret._sync_copyfrom(summed)
    row_ret = empty(indptr.shape, ctx)
    row_ret._sync_copyfrom(indptr, np.int32)
    col_ret = empty(ucols.shape, ctx)
    col_ret._sync_copyfrom(ucols, np.int32)
    return ND_Sparse_Array(values_ret, row_ret, col_ret, int(shape[0]), int(shape[1]))


def numpyasdlarrayhandle(data):
    arr, shape = NDArray._numpyasarray(np.ascontiguousarray(data, dtype=np.float32))
    arr._keep = shape
    return arr


def tensor_reuse(input_shape, output_shape, pieces, overlap_pieces, ctx=gpu(0)):
    """(input, output) sharing one allocation: output at the base, input flush with the end,
    overlapping by `overlap_pieces` of the input's `pieces` micro-tensors.  The output owns
    the allocation; the input is a view of it."""
    ih, oh = DLArrayHandle(), DLArrayHandle()
    ishape = c_array(ctypes.c_int64, tuple(input_shape))
    oshape = c_array(ctypes.c_int64, tuple(output_shape))
    check_call(_LIB.DLArrayReuseAlloc(ctx, ctypes.c_int(MEMORY_MANAGE_RULE),
                                      ishape, ctypes.c_int64(len(ishape)), ctypes.byref(ih),
                                      oshape, ctypes.c_int64(len(oshape)), ctypes.byref(oh),
                                      ctypes.c_int(pieces), ctypes.c_int(overlap_pieces)))
    output_arr = NDArray(oh)                       # data pointer == allocation base
    input_arr = NDArray(ih, owner=output_arr, is_view=True)
    return input_arr, output_arr


def slice_for_micro_tensor(input_tensor, index, total_number, dimension="batch"):
    if dimension == "batch":
        dim = 0
    elif dimension == "channel":
        dim = 1
    else:
        raise NotImplementedError
    h = DLArrayHandle()
    check_call(_LIB.DLArraySliceForMicroTensor(input_tensor.handle, ctypes.byref(h),
                                               ctypes.c_int(total_number), ctypes.c_int(index),
                                               ctypes.c_int(dim)))
    return NDArray(h, auto_deleted=False, owner=input_tensor, is_view=True)


def split_shape(input_shape, total_number=0, dimension="batch"):
    assert total_number > 0
    d = 0 if dimension == "batch" else 1
    base, extra = input_shape[d] // total_number, input_shape[d] % total_number
    out = []
    for idx in range(total_number):
        s = list(input_shape)
        s[d] = base + (1 if idx < extra else 0)
        out.append(s)
    return out
