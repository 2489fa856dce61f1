"""Empty tensors (a batch of zero images, zero rows): data-movement, elementwise, pooling,
convolution and matrix-product entry points accept them and do nothing; a product over an empty
reduction writes zeros; reductions that would divide by zero (BatchNorm statistics, the mean
cross-entropy) refuse with an error instead of launching anything.  Nothing crashes."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _env():
    from tsplit_amd import gpu_links as L, ndarray as nd
    return L, nd, nd.gpu(0)


def test_elementwise_and_layout_ops_on_empty_arrays():
    L, nd, ctx = _env()
    e = lambda *s: nd.empty(tuple(s), ctx)
    a, b, c = e(0, 8, 4, 4), e(0, 8, 4, 4), e(0, 8, 4, 4)
    L.relu(a, c)
    L.relu_gradient(a, b, c)
    L.matrix_elementwise_add(a, b, c)
    L.matrix_elementwise_multiply(a, b, c)
    L.matrix_elementwise_add_by_const(a, 1.0, c)
    L.matrix_elementwise_multiply_by_const(a, 2.0, c)
    L.array_set(c, 3.0)
    L.sigmoid(a, c)
    L.tanh(a, c)
    L.array_reshape(a, e(0, 128))
    L.matrix_transpose(a, e(4, 4, 8, 0), (3, 2, 1, 0))
    L.concat(a, b, e(0, 16, 4, 4), 1)
    L.concat(e(2, 0, 4, 4), e(2, 3, 4, 4), e(2, 3, 4, 4), 1)
    L.concat_gradient(e(0, 16, 4, 4), a, 1, 0)
    L.matrix_slice(e(0, 16, 4, 4), a, [0, 8, 0, 0])
    L.sgd_update(e(0,), e(0,), 0.1)
    L.momentum_update(e(0,), e(0,), e(0,), 0.1, 0.9, False)
    L.adam_update(e(0,), e(0,), e(0,), e(0,), 0.1, 0.9, 0.999, 0.9, 0.999, 1e-8)
    assert c.asnumpy().shape == (0, 8, 4, 4)


def test_pooling_and_convolution_on_an_empty_batch():
    L, nd, ctx = _env()
    e = lambda *s: nd.empty(tuple(s), ctx)
    x, y = e(0, 16, 8, 8), e(0, 16, 4, 4)
    L.max_pooling2d(x, 2, 2, y, 0, 2)
    L.max_pooling2d_gradient(x, y, 2, 2, e(0, 16, 8, 8), 0, 2)
    L.CuDNN_max_pooling2d(x, 2, 2, y, 0, 2)
    L.average_pooling2d(x, 2, 2, y, 0, 2)
    L.average_pooling2d_gradient(y, 2, 2, e(0, 16, 8, 8), 0, 2)
    w = nd.array(np.ones((32, 16, 3, 3), np.float32), ctx)
    out, dx = e(0, 32, 8, 8), e(0, 16, 8, 8)
    L.CuDNN_conv2d(x, w, out, 1, 1, 1)
    L.CuDNN_conv2d_gradient_of_data(w, out, dx, 1, 1, 1)
    # the filter gradient over an empty batch is a sum of nothing
    dw = nd.array(np.full((32, 16, 3, 3), 7.0, np.float32), ctx)
    L.CuDNN_conv2d_gradient_of_filter(x, out, dw, 1, 1, 1)
    assert not dw.asnumpy().any()
    # every route of the dispatcher: a first layer on 3 channels (1x1 stride 2 and 3x3), a 1x1 and a strided layer on
    # many channels, a channel count that is no multiple of 16, a layer the Winograd routine would take
    for (C, O, k, pad, s, H) in [(3, 24, 1, 0, 2, 12), (3, 64, 3, 1, 1, 16), (64, 256, 1, 0, 1, 8), (32, 48, 3, 1, 2, 9),
                                 (20, 10, 5, 2, 1, 7), (64, 64, 3, 1, 1, 64)]:
        oH = (H + 2 * pad - k) // s + 1
        x, y, dx = e(0, C, H, H), e(0, O, oH, oH), e(0, C, H, H)
        w = nd.array(np.ones((O, C, k, k), np.float32), ctx)
        dw = nd.array(np.full((O, C, k, k), 7.0, np.float32), ctx)
        L.CuDNN_conv2d(x, w, y, pad, pad, s)
        L.CuDNN_conv2d_gradient_of_data(w, y, dx, pad, pad, s)
        L.CuDNN_conv2d_gradient_of_filter(x, y, dw, pad, pad, s)
        assert not dw.asnumpy().any(), (C, O, k, pad, s, H)


def test_matrix_products_with_an_empty_dimension():
    L, nd, ctx = _env()
    e = lambda *s: nd.empty(tuple(s), ctx)
    L.matrix_multiply(e(0, 16), False, e(16, 8), False, e(0, 8))
    L.matrix_multiply(e(4, 16), False, e(16, 0), False, e(4, 0))
    c = nd.array(np.full((4, 8), 5.0, np.float32), ctx)
    L.matrix_multiply(e(4, 0), False, e(0, 8), False, c)          # empty reduction: zeros
    assert not c.asnumpy().any()
    L.batch_matrix_multiply(e(0, 4, 16), False, e(0, 16, 8), False, e(0, 4, 8))


def test_reductions_over_nothing_are_refused():
    L, nd, ctx = _env()
    e = lambda *s: nd.empty(tuple(s), ctx)
    g = nd.array(np.ones((1, 8, 1, 1), np.float32), ctx)
    with pytest.raises(RuntimeError):
        L.CuDNN_Batch_Normalization(e(0, 8, 4, 4), g, g, e(0, 8, 4, 4), None, None, 0.99, 0.01)
    with pytest.raises(RuntimeError):
        L.softmax_cross_entropy(e(0, 10), e(0, 10), e(1,))
    # and afterwards the library still works
    x = nd.array(np.array([[-1.0, 2.0]], np.float32), ctx)
    y = nd.empty((1, 2), ctx)
    L.relu(x, y)
    assert y.asnumpy().tolist() == [[0.0, 2.0]]
