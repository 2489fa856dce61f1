"""Invalid calls return -1 (raised as RuntimeError by the wrappers) where the reference asserts, reads
out of bounds or exits (src/common/runtime_base.h:18-47, src/cuda_common/gpu_runtime.h:21-43); nothing
is launched, and the library keeps working afterwards."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_shape_violations_are_refused():
    from tsplit_amd import gpu_links as L, ndarray as nd
    ctx = nd.gpu(0)
    e = lambda *s: nd.empty(tuple(s), ctx)
    bad = [
        lambda: L.CuDNN_conv2d(e(2, 16, 8, 8), e(4, 16, 3, 3), e(2, 4, 7, 7), 1, 1, 1),          # output should be 8x8
        lambda: L.CuDNN_conv2d(e(2, 16, 8, 8), e(4, 8, 3, 3), e(2, 4, 8, 8), 1, 1, 1),           # filter channels
        lambda: L.CuDNN_conv2d(e(2, 16, 2, 2), e(4, 16, 5, 5), e(2, 4, 1, 1), 0, 0, 1),          # filter larger than the image
        lambda: L.CuDNN_conv2d_gradient_of_data(e(4, 16, 3, 3), e(2, 5, 8, 8), e(2, 16, 8, 8), 1, 1, 1),
        lambda: L.CuDNN_conv2d_gradient_of_filter(e(2, 16, 8, 8), e(2, 4, 8, 8), e(4, 16, 5, 5), 1, 1, 1),
        lambda: L.CuDNN_Batch_Normalization(e(2, 8, 4, 4), e(1, 7, 1, 1), e(1, 8, 1, 1), e(2, 8, 4, 4), None, None, 0.99, 0.01),
        lambda: L.CuDNN_Batch_Normalization(e(2, 8, 16), e(1, 8, 1, 1), e(1, 8, 1, 1), e(2, 8, 16), None, None, 0.99, 0.01),
        lambda: L.max_pooling2d(e(2, 3, 8, 8), 2, 2, e(2, 3, 5, 5), 0, 2),
        lambda: L.matrix_multiply(e(4, 5), True, e(4, 3), False, e(4, 3)),
        lambda: L.batch_matrix_multiply(e(2, 4, 5), False, e(3, 5, 6), False, e(2, 4, 6)),
        lambda: L.concat(e(2, 3, 4), e(2, 5, 5), e(2, 8, 4), 1),
        lambda: L.concat(e(2, 3, 4), e(2, 5, 4), e(2, 9, 4), 1),
        lambda: L.matrix_slice(e(4, 4), e(3, 3), [2, 0]),                                          # window leaves the tensor
        lambda: L.softmax_cross_entropy(e(4, 10), e(4, 9), e(1,)),
        lambda: L.matrix_transpose(e(2, 3, 4), e(4, 3, 2), (0, 1, 1)),                             # not a permutation
        lambda: L.reduce_sum(e(2, 3, 4), e(2, 4), [5]),
        lambda: L.pad(e(1, 1, 4, 4), e(1, 1, 6, 7), [(1, 1), (1, 1)], "CONSTANT", 0.0),
        lambda: L.embedding_lookup(e(10, 4), e(3,), e(3, 5)),
    ]
    for i, call in enumerate(bad):
        with pytest.raises(RuntimeError):
            call()
            pytest.fail("call %d was accepted" % i)
    x = nd.array(np.arange(6, dtype=np.float32).reshape(2, 3) - 2, ctx)
    y = nd.empty((2, 3), ctx)
    L.relu(x, y)
    assert y.asnumpy().tolist() == [[0, 0, 0], [1, 2, 3]]


def test_runtime_calls_report_errors():
    import ctypes
    from tsplit_amd import ndarray as nd
    from tsplit_amd._base import _LIB
    a, b = nd.empty((4,), nd.gpu(0)), nd.empty((5,), nd.gpu(0))
    assert _LIB.DLArrayCopyFromTo(a.handle, b.handle, None) == -1          # sizes differ
    assert _LIB.DLEventRecord(None, None) == -1
    assert _LIB.DLEventSync(None) == -1
    assert _LIB.DLEventQuery(None) == 0
    out = nd.DLArrayHandle()
    assert _LIB.DLArraySliceForMicroTensor(a.handle, ctypes.byref(out), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)) == -1
    assert _LIB.DLArraySliceForMicroTensor(a.handle, ctypes.byref(out), ctypes.c_int(2), ctypes.c_int(2), ctypes.c_int(0)) == -1
