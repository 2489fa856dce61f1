"""GPU parity of the operators around the core path (average pooling, broadcast / reduce,
pad, transpose, batched matmul, one-hot, where, embedding, elementwise math) against the CPU
oracle, called through the C ABI.  Tolerances: bit-exact for pure data movement (broadcast,
pad, transpose, one-hot, where, embedding lookup); 1e-4 max relative error for sums and
elementwise math; 2e-3 for batched matmul."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 1e-4
TOL_MM = 2e-3


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


AVG_CASES = [
    # N, C, H, W, kH, kW, pad, stride
    (4, 64, 7, 7, 7, 7, 0, 7),       # ResNet-50 global pool (channels cut down)
    (2, 48, 8, 8, 8, 8, 0, 1),       # Inception-v4 global pool
    (2, 24, 35, 35, 3, 3, 1, 1),     # Inception-A 3x3 same pool
    (2, 16, 17, 17, 3, 3, 1, 1),
    (1, 3, 9, 11, 3, 2, 1, 2),       # ragged, floors, non-square window
    (2, 5, 12, 12, 2, 2, 0, 2),
    (1, 2, 5, 5, 5, 5, 2, 1),        # every window clipped
]


@pytest.mark.parametrize("case", AVG_CASES)
@pytest.mark.parametrize("family", ["plain", "cudnn"])
def test_avg_pool_forward_backward(ts, case, family, rng):
    N, C, H, W, kH, kW, pad, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    ref = O.avg_pool(x, kH, kW, pad, s)
    dy = rng.normal(size=ref.shape).astype(np.float32)
    gx, gy, gdy, gdx = ts.arr(x), ts.empty(ref.shape), ts.arr(dy), ts.empty(x.shape)
    L = ts.links
    if family == "plain":
        L.average_pooling2d(gx, kH, kW, gy, pad, s, ts.stream)
        L.average_pooling2d_gradient(gdy, kH, kW, gdx, pad, s, ts.stream)
    else:
        L.CuDNN_average_pooling2d(gx, kH, kW, gy, pad, s, ts.stream)
        L.CuDNN_average_pooling2d_gradient(gy, gdy, gx, kH, kW, gdx, pad, s, ts.stream)
    assert_close(gy.asnumpy(), ref, TOL, "avg_pool")
    assert_close(gdx.asnumpy(), O.avg_pool_grad(dy, x.shape, kH, kW, pad, s), TOL, "avg_pool_grad")


def test_avg_pool_rejects_wrong_output_shape(ts):
    x, y = ts.empty((1, 1, 8, 8)), ts.empty((1, 1, 3, 3))
    with pytest.raises(RuntimeError):
        ts.links.average_pooling2d(x, 2, 2, y, 0, 2, ts.stream)


@pytest.mark.parametrize("in_shape,out_shape", [((10,), (128, 10)), ((1000,), (64, 1000)), ((7,), (5, 7)),
                                                ((3, 5), (4, 3, 5)), ((512,), (32, 256, 512)), ((1,), (9,))])
def test_broadcast_to_and_reduce_sum_axis_zero(ts, in_shape, out_shape, rng):
    b = rng.normal(size=in_shape).astype(np.float32)
    out = ts.empty(out_shape)
    ts.links.broadcast_to(ts.arr(b), out, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.broadcast_to(b, out_shape).astype(np.float32))
    x = rng.normal(size=out_shape).astype(np.float32)
    lead = int(np.prod(out_shape)) // int(np.prod(in_shape))
    x2 = x.reshape((lead,) + in_shape)
    r = ts.empty(in_shape)
    ts.links.reduce_sum_axis_zero(ts.arr(x2), r, ts.stream)
    assert_close(r.asnumpy(), O.reduce_sum_axis_zero(x2), TOL, "reduce_sum_axis_zero")
    ws = ts.empty(x2.shape)
    r2 = ts.empty(in_shape)
    ts.links._reduce_sum_axis_zero(ts.arr(x2), r2, ws, ts.stream)
    np.testing.assert_array_equal(r2.asnumpy(), r.asnumpy())


@pytest.mark.parametrize("rows,cols", [(8192, 512), (3, 100003), (1, 17), (70000, 3), (257, 1024)])
def test_reduce_sum_axis_zero_shapes(ts, rows, cols, rng):
    x = rng.normal(size=(rows, cols)).astype(np.float32)
    r = ts.empty((cols,))
    ts.links.reduce_sum_axis_zero(ts.arr(x), r, ts.stream)
    assert_close(r.asnumpy(), O.reduce_sum_axis_zero(x), TOL, "reduce_sum_axis_zero")


@pytest.mark.parametrize("shape", [(2, 3, 4, 5), (8, 64, 56, 56), (4, 96, 35, 35), (16, 2048, 7, 7), (1, 1, 1, 1),
                                   (64, 8, 112, 112)])
def test_conv_bias_broadcast_and_reduce(ts, shape, rng):
    b = rng.normal(size=(shape[1],)).astype(np.float32)
    out = ts.empty(shape)
    ts.links.conv2d_broadcast_to(ts.arr(b), out, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.conv2d_broadcast_to(b, shape).astype(np.float32))
    x = rng.normal(size=shape).astype(np.float32)
    r = ts.empty((shape[1],))
    ts.links.conv2d_reduce_sum(ts.arr(x), r, ts.stream)
    assert_close(r.asnumpy(), O.conv2d_reduce_sum(x), TOL, "conv2d_reduce_sum")


@pytest.mark.parametrize("in_shape,out_shape,add_axes", [
    ((256, 256), (4, 8, 256, 256), None),    # causal mask of the transformer
    ((3, 1, 4), (2, 3, 5, 4), None),
    ((2, 4), (2, 3, 4), [1]),
    ((3,), (2, 3, 4), [0, 2]),
    ((2, 3), (2, 5, 3, 4), [1, 3]),
    ((32, 1, 1, 256), (32, 8, 256, 256), None),
    ((5, 1), (5, 7), None),
])
def test_broadcast_shape(ts, in_shape, out_shape, add_axes, rng):
    x = rng.normal(size=in_shape).astype(np.float32)
    out = ts.empty(out_shape)
    ts.links.broadcast_shape(ts.arr(x), out, add_axes, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.broadcast_shape(x, out_shape, add_axes).astype(np.float32))


@pytest.mark.parametrize("shape,axes", [
    ((32, 255, 64), [0, 1]), ((32, 255, 64), [2]), ((32, 255, 64), [1]), ((32, 255, 64), [0, 2]),
    ((4, 8, 256, 256), [0, 1]), ((4, 8, 64, 64), [3]), ((3, 4, 5, 2), [0, 1, 2, 3]), ((6, 1, 7), [1]),
    ((2, 3, 4, 5, 6), [1, 3]), ((100003,), [0]), ((5, 100003), [1]), ((64, 3, 9), [0, 2]),
])
def test_reduce_sum(ts, shape, axes, rng):
    x = rng.normal(size=shape).astype(np.float32)
    ref = O.reduce_sum(x, axes)
    for keep in (False, True):
        oshape = O.reduce_sum(x, axes, keepdims=keep).shape or (1,)
        out = ts.empty(oshape)
        ts.links.reduce_sum(ts.arr(x), out, axes, ts.stream)
        assert_close(out.asnumpy().reshape(ref.shape), ref, TOL, "reduce_sum")


@pytest.mark.parametrize("shape,paddings", [
    ((2, 3, 4, 5), [(1, 1), (1, 1)]),
    ((2, 3, 8, 8), [(0, 2), (4, 0)]),          # word-aligned padding along W
    ((2, 3, 4, 5), [(1, 0), (0, 0), (2, 1)]),
    ((2, 3, 4, 5), [(1, 1), (0, 1), (1, 0), (2, 2)]),
    ((4, 16, 35, 35), [(0, 1), (0, 1)]),
    ((2, 3, 6, 8), []),
])
def test_pad_and_gradient(ts, shape, paddings, rng):
    x = rng.normal(size=shape).astype(np.float32)
    ref = O.pad(x, paddings, 0.5)
    out = ts.empty(ref.shape)
    ts.links.pad(ts.arr(x), out, paddings, "CONSTANT", 0.5, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), ref.astype(np.float32))
    dy = rng.normal(size=ref.shape).astype(np.float32)
    dx = ts.empty(shape)
    ts.links.pad_gradient(ts.arr(dy), dx, paddings, "CONSTANT", ts.stream)
    np.testing.assert_array_equal(dx.asnumpy(), O.pad_grad(dy, paddings).astype(np.float32))


def test_pad_rejects_other_modes(ts):
    x, y = ts.empty((1, 1, 4, 4)), ts.empty((1, 1, 6, 6))
    with pytest.raises(RuntimeError):
        ts.links.pad(x, y, [(1, 1), (1, 1)], "REFLECT", 0.0, ts.stream)


@pytest.mark.parametrize("shape,perm", [
    ((32, 256, 8, 64), (0, 2, 1, 3)),      # transformer split-heads
    ((32, 8, 256, 64), (0, 2, 1, 3)),      # and back
    ((300, 500), (1, 0)), ((64, 64), (1, 0)), ((1000, 3), (1, 0)), ((3, 1000), (1, 0)),
    ((2, 3, 4, 5), (3, 2, 1, 0)), ((6, 70, 130), (0, 2, 1)), ((6, 70, 130), (2, 0, 1)), ((6, 70, 130), (1, 2, 0)),
    ((2, 3, 4), (0, 1, 2)), ((5, 7, 9, 11), (2, 3, 0, 1)), ((4, 1, 33, 65), (3, 1, 0, 2)),
])
def test_transpose(ts, shape, perm, rng):
    x = rng.normal(size=shape).astype(np.float32)
    ref = O.transpose(x, perm)
    out = ts.empty(ref.shape)
    ts.links.matrix_transpose(ts.arr(x), out, perm, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), ref)


@pytest.mark.parametrize("lead,M,N,K", [((4, 8), 256, 256, 64), ((4, 8), 256, 64, 256), ((3,), 70, 50, 33),
                                        ((2, 2), 64, 300, 17), ((5,), 1, 1, 1), ((2,), 130, 40, 128)])
@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
def test_batch_matmul(ts, lead, M, N, K, tA, tB, rng):
    A = rng.normal(size=lead + ((K, M) if tA else (M, K))).astype(np.float32)
    B = rng.normal(size=lead + ((N, K) if tB else (K, N))).astype(np.float32)
    out = ts.empty(lead + (M, N))
    ts.links.batch_matrix_multiply(ts.arr(A), tA, ts.arr(B), tB, out, ts.stream)
    assert_close(out.asnumpy(), O.batch_matmul(A, tA, B, tB), TOL_MM, "batch_matmul")


def test_one_hot_where_embedding(ts, rng):
    ids = rng.randint(0, 1000, size=(8, 33)).astype(np.float32)
    for classes in (1000, 1001):
        out = ts.empty(ids.shape + (classes,))
        ts.links.one_hot(ts.arr(ids), out, ts.stream)
        np.testing.assert_array_equal(out.asnumpy(), O.one_hot(ids, classes))
    c = (rng.rand(8, 33, 5) > 0.5).astype(np.float32)
    a, b = rng.normal(size=c.shape).astype(np.float32), rng.normal(size=c.shape).astype(np.float32)
    out = ts.empty(c.shape)
    ts.links.where(ts.arr(c), ts.arr(a), ts.arr(b), out, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.where(c, a, b))
    for width in (512, 30):
        table = rng.normal(size=(1000, width)).astype(np.float32)
        e = ts.empty(ids.shape + (width,))
        ts.links.embedding_lookup(ts.arr(table), ts.arr(ids), e, ts.stream)
        np.testing.assert_array_equal(e.asnumpy(), O.embedding_lookup(table, ids))
        dy = rng.normal(size=ids.shape + (width,)).astype(np.float32)
        g = ts.empty(table.shape)
        ts.links.array_set(g, 7.0, ts.stream)               # the gradient zero-fills its output itself
        ts.links.embedding_lookup_gradient(ts.arr(dy), ts.arr(ids), g, ts.stream)
        assert_close(g.asnumpy(), O.embedding_lookup_grad(dy, ids, table.shape), TOL, "embedding_grad")


def test_embedding_ids_outside_the_table_read_zero_and_add_nothing(ts, rng):
    table = rng.normal(size=(10, 8)).astype(np.float32)
    ids = np.array([[0, 9, 10, -3]], np.float32)
    e = ts.empty((1, 4, 8))
    ts.links.embedding_lookup(ts.arr(table), ts.arr(ids), e, ts.stream)
    got = e.asnumpy()
    np.testing.assert_array_equal(got[0, :2], table[[0, 9]])
    assert np.all(got[0, 2:] == 0)
    dy = np.ones((1, 4, 8), np.float32)
    g = ts.empty(table.shape)
    ts.links.embedding_lookup_gradient(ts.arr(dy), ts.arr(ids), g, ts.stream)
    ref = np.zeros_like(table)
    ref[[0, 9]] = 1
    np.testing.assert_array_equal(g.asnumpy(), ref)


@pytest.mark.parametrize("shape", [(5,), (4097,), (32, 255, 64)])
def test_elementwise_math(ts, shape, rng):
    x = (rng.rand(*shape) * 4 + 0.1).astype(np.float32)
    z = (rng.normal(size=shape) * 3).astype(np.float32)
    z.ravel()[:3] = [-100.0, 100.0, 0.0][:min(3, z.size)]
    gx, gz, out = ts.arr(x), ts.arr(z), ts.empty(shape)
    L, s = ts.links, ts.stream
    L.matrix_sqrt(gx, out, s); assert_close(out.asnumpy(), O.sqrt(x), TOL, "sqrt")
    L.matrix_rsqrt(gx, out, s); assert_close(out.asnumpy(), O.rsqrt(x), TOL, "rsqrt")
    L.sigmoid(gz, out, s); assert_close(out.asnumpy(), O.sigmoid(z), TOL, "sigmoid")
    L.tanh(gz, out, s); assert_close(out.asnumpy(), O.tanh(z), TOL, "tanh")
    L.matrix_opposite(gz, out, s); np.testing.assert_array_equal(out.asnumpy(), O.opposite(z).astype(np.float32))
    L.matrix_elementwise_divide_const(3.0, gx, out, s); assert_close(out.asnumpy(), O.div_const(3.0, x), TOL, "div_const")
    L.matrix_elementwise_divide(gz, gx, out, s); assert_close(out.asnumpy(), O.divide(z, x), TOL, "divide")


def test_profiler_is_filled_for_a_wider_op(ts, rng):
    from tsplit_amd import profiler
    x = rng.normal(size=(4, 16, 35, 35)).astype(np.float32)
    y = ts.empty((4, 16, 35, 35))
    p = profiler.CreateProfiler()
    ts.links.average_pooling2d(ts.arr(x), 3, 3, y, 1, 1, ts.stream, p)
    assert p.time >= 0 and abs(p.input_memory - x.size * 4 / 2 ** 20) < 1e-3 and p.workspace_memory == 0
