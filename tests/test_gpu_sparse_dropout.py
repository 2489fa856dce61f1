"""GPU parity of dropout and the CSR sparse products against the CPU oracle, through the C ABI.

Dropout is compared bit for bit (mask and values) with the oracle's float32 evaluation; its
mask is this library's Philox stream, pinned on the CPU side by the published known-answer
vectors.  Sparse products: max relative error 1e-4 against the float64 oracle (sums of up
to a few hundred products per output)."""
import ctypes

import numpy as np
import pytest
import scipy.sparse

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def ts():
    from tsplit_amd import gpu_links, ndarray, stream
    ctx = ndarray.gpu(0)

    class NS:
        pass
    ns = NS()
    ns.links, ns.nd, ns.ctx = gpu_links, ndarray, ctx
    ns.stream = stream.create_stream_handle(ctx)
    ns.arr = lambda a: ndarray.array(np.asarray(a, np.float32), ctx)
    ns.empty = lambda shape: ndarray.empty(shape, ctx)
    return ns


DROPOUT_SHAPES = [(1,), (7,), (8,), (9,), (1000,), (4099,), (4, 3, 5, 7), (128, 1000), (3, 2**18 + 3)]


@pytest.mark.parametrize("shape", DROPOUT_SHAPES)
@pytest.mark.parametrize("p", [0.1, 0.5])
def test_dropout_forward_gradient_bit_exact(ts, shape, p, rng):
    x = (rng.normal(size=shape) + 3.0).astype(np.float32)
    dy = rng.normal(size=shape).astype(np.float32)
    want, keep = O.dropout(x, p, dtype=np.float32)
    gx, gy, gdy, gdx = ts.arr(x), ts.empty(shape), ts.arr(dy), ts.empty(shape)
    size, space = ctypes.c_int(0), ctypes.c_void_p(0)
    ts.links.CuDNN_Dropout(gx, p, gy, size, space, 1, ts.stream)
    ts.stream.sync()
    assert size.value == (x.size + 7) // 8 and space.value
    got = gy.asnumpy()
    assert np.array_equal(got != 0, keep)
    assert np.array_equal(got, want)
    # later calls reuse the reserve space and repeat the mask (the generator is re-seeded)
    first_space = space.value
    gy2 = ts.empty(shape)
    ts.links.CuDNN_Dropout(gx, p, gy2, size, space, 0, ts.stream)
    ts.links.CuDNN_Dropout_gradient(gdy, p, gdx, size, space, ts.stream)
    ts.stream.sync()
    assert space.value == first_space
    assert np.array_equal(gy2.asnumpy(), want)
    assert np.array_equal(gdx.asnumpy(), O.dropout_grad(dy, p, keep, dtype=np.float32))


def test_dropout_unaligned_views_and_extremes(ts, rng):
    """Rows of 5 floats cut into micro-tensors start 20 bytes apart: the scalar path."""
    x = (rng.normal(size=(3, 5)) + 3.0).astype(np.float32)
    gx, gy = ts.arr(x), ts.empty((3, 5))
    gx.split_tensor(3)
    gy.split_tensor(3)
    xs, ys = gx.sTensor, gy.sTensor
    for i in range(3):
        size, space = ctypes.c_int(0), ctypes.c_void_p(0)
        ts.links.CuDNN_Dropout(xs[i], 0.5, ys[i], size, space, 1, ts.stream)
    ts.stream.sync()
    got = gy.asnumpy()
    for i in range(3):
        keep = O.dropout_mask(5, 0.5)
        assert np.array_equal(got[i] != 0, keep)
        assert np.array_equal(got[i], np.where(keep, x[i] * np.float32(2.0), np.float32(0)))
    # p = 0 keeps everything unchanged, p = 1 clears everything
    big = (rng.normal(size=(1000,)) + 3.0).astype(np.float32)
    gb, go = ts.arr(big), ts.empty((1000,))
    size, space = ctypes.c_int(0), ctypes.c_void_p(0)
    ts.links.CuDNN_Dropout(gb, 0.0, go, size, space, 1, ts.stream)
    ts.stream.sync()
    assert np.array_equal(go.asnumpy(), big)
    ts.links.CuDNN_Dropout(gb, 1.0, go, size, space, 0, ts.stream)
    ts.stream.sync()
    assert np.all(go.asnumpy() == 0)


def test_dropout_transformer_size_properties(ts, rng):
    """At the Transformer activation size [32, 256, 512]: dropped fraction within five standard
    deviations, dropout(2x) == 2 dropout(x) exactly, and gradient(dy = x) == forward(x)."""
    shape, p = (32, 256, 512), 0.3
    x = (rng.normal(size=shape) + 4.0).astype(np.float32)
    gx, gy, g2, gd = ts.arr(x), ts.empty(shape), ts.empty(shape), ts.empty(shape)
    size, space = ctypes.c_int(0), ctypes.c_void_p(0)
    ts.links.CuDNN_Dropout(gx, p, gy, size, space, 1, ts.stream)
    ts.links.CuDNN_Dropout_gradient(gx, p, gd, size, space, ts.stream)
    gx2 = ts.arr(2 * x)
    ts.links.CuDNN_Dropout(gx2, p, g2, size, space, 0, ts.stream)
    ts.stream.sync()
    y = gy.asnumpy()
    n = x.size
    dropped = float((y == 0).mean())
    assert abs(dropped - p) <= 5 * np.sqrt(p * (1 - p) / n)
    assert np.array_equal(g2.asnumpy(), 2 * y)
    assert np.array_equal(gd.asnumpy(), y)
    assert np.array_equal(y != 0, O.dropout_mask(n, p).reshape(shape))


def test_dropout_rejects_bad_arguments(ts):
    gx, gy, gz = ts.empty((4, 4)), ts.empty((4, 4)), ts.empty((4, 5))
    size, space = ctypes.c_int(0), ctypes.c_void_p(0)
    with pytest.raises(RuntimeError):
        ts.links.CuDNN_Dropout(gx, 0.5, gz, size, space, 1, ts.stream)           # shapes differ
    with pytest.raises(RuntimeError):
        ts.links.CuDNN_Dropout(gx, 1.5, gy, size, space, 1, ts.stream)           # not a probability
    with pytest.raises(RuntimeError):
        ts.links.CuDNN_Dropout(gx, 0.5, gy, size, space, 0, ts.stream)           # no reserve space yet
    with pytest.raises(RuntimeError):
        ts.links.CuDNN_Dropout_gradient(gx, 0.5, gy, size, space, ts.stream)


def _random_csr(rng, nrow, ncol, density, empty_rows=()):
    m = scipy.sparse.random(nrow, ncol, density=density, format="csr", dtype=np.float32,
                            random_state=rng, data_rvs=lambda k: rng.normal(size=k).astype(np.float32))
    if empty_rows:
        m = m.tolil()
        for r in empty_rows:
            m[r, :] = 0
        m = m.tocsr()
    m.eliminate_zeros()
    m.sort_indices()
    return m


def _upload(ts, m):
    coo = m.tocoo()
    return ts.nd.sparse_array(coo.data, (coo.row, coo.col), m.shape, ts.ctx)


CSR_CASES = [
    # nrow, ncol, density, empty rows
    (5, 7, 0.4, ()),
    (100, 80, 0.1, (0, 17, 99)),
    (1000, 1200, 0.01, ()),         # ~12 entries per row
    (64, 3000, 0.12, (5,)),         # ~360 entries per row: a whole wave per row
    (3000, 50, 0.02, ()),           # ~1 entry per row
    (1, 1, 1.0, ()),
]


@pytest.mark.parametrize("case", CSR_CASES)
@pytest.mark.parametrize("trans", [False, True])
def test_csrmv(ts, case, trans, rng):
    nrow, ncol, density, empty = case
    m = _random_csr(rng, nrow, ncol, density, empty)
    A = _upload(ts, m)
    x = rng.normal(size=nrow if trans else ncol).astype(np.float32)
    gx, gy = ts.arr(x), ts.empty((ncol if trans else nrow,))
    ts.links.CuSparse_Csrmv(A, trans, gx, gy, ts.stream)
    ts.stream.sync()
    assert_close(gy.asnumpy(), O.csrmv(m.data, m.indptr, m.indices, nrow, ncol, trans, x), TOL, "csrmv")


@pytest.mark.parametrize("case", CSR_CASES)
@pytest.mark.parametrize("n", [1, 3, 16, 100])
@pytest.mark.parametrize("transA,transB", [(False, False), (True, False), (False, True), (True, True)])
def test_csrmm(ts, case, n, transA, transB, rng):
    nrow, ncol, density, empty = case
    m = _random_csr(rng, nrow, ncol, density, empty)
    A = _upload(ts, m)
    inner, outer = (nrow, ncol) if transA else (ncol, nrow)
    B = rng.normal(size=(n, inner) if transB else (inner, n)).astype(np.float32)
    gB, gC = ts.arr(B), ts.empty((outer, n))
    ts.links.CuSparse_Csrmm(A, transA, gB, transB, gC, ts.stream)
    ts.stream.sync()
    assert_close(gC.asnumpy(), O.csrmm(m.data, m.indptr, m.indices, nrow, ncol, transA, B, transB), TOL, "csrmm")


def test_csr_upload_sums_duplicates_and_empty_matrix(ts, rng):
    vals = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    rows, cols = np.array([2, 0, 2, 0]), np.array([1, 3, 1, 0])
    A = ts.nd.sparse_array(vals, (rows, cols), (3, 4), ts.ctx)
    assert A.shape == (3, 4) and A.data.shape == (3,)
    x = np.array([1.0, 10.0, 100.0, 1000.0], np.float32)
    gy = ts.empty((3,))
    ts.links.CuSparse_Csrmv(A, False, ts.arr(x), gy, ts.stream)
    ts.stream.sync()
    assert np.array_equal(gy.asnumpy(), np.array([2004.0, 0.0, 40.0], np.float32))
    # a matrix without entries gives zeros, also in the scattering (transposed) form
    Z = ts.nd.sparse_array(np.zeros(0, np.float32), (np.zeros(0, int), np.zeros(0, int)), (3, 4), ts.ctx)
    gz = ts.arr(np.full((4,), 7.0, np.float32))
    ts.links.CuSparse_Csrmv(Z, True, ts.arr(np.ones(3, np.float32)), gz, ts.stream)
    ts.stream.sync()
    assert np.all(gz.asnumpy() == 0)


def test_csr_rejects_bad_shapes(ts):
    A = ts.nd.sparse_array(np.ones(2, np.float32), (np.array([0, 1]), np.array([1, 0])), (2, 2), ts.ctx)
    with pytest.raises(RuntimeError):
        ts.links.CuSparse_Csrmv(A, False, ts.empty((3,)), ts.empty((2,)), ts.stream)
    with pytest.raises(RuntimeError):
        ts.links.CuSparse_Csrmm(A, False, ts.empty((3, 4)), False, ts.empty((2, 4)), ts.stream)
    bad = ts.nd.ND_Sparse_Array(A.data, A.col, A.col, 2, 2)      # row pointer array of the wrong length
    with pytest.raises(RuntimeError):
        ts.links.CuSparse_Csrmv(bad, False, ts.empty((2,)), ts.empty((2,)), ts.stream)
