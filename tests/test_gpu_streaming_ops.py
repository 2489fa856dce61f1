"""GPU parity of the HBM-streaming operators against the CPU oracle, called through the
C ABI (tsplit_amd.gpu_links -> libc_runtime_api.so).  Tolerances: 1e-4 max relative error
for elementwise / BN / softmax results; bit-exact for pooling, split, concat, slice."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close, assert_close_entries

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.fixture(scope="module")
def ts():
    import tsplit_amd
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


SIZES = [1, 3, 4, 1023, 4096, 4097, 100003, (2, 3, 5, 7), (16, 64, 56, 56)]


@pytest.mark.parametrize("shape", SIZES)
def test_elementwise_family(ts, shape, rng):
    shape = (shape,) if isinstance(shape, int) else shape
    a = rng.normal(size=shape).astype(np.float32)
    b = rng.normal(size=shape).astype(np.float32)
    a.ravel()[::7] = 0.0                      # exercise relu'(0) = 0.5
    ga, gb, out = ts.arr(a), ts.arr(b), ts.empty(shape)
    L, s = ts.links, ts.stream
    L.matrix_elementwise_add(ga, gb, out, s); assert_close_entries(out.asnumpy(), O.add(a, b), TOL, "add")
    L.matrix_elementwise_multiply(ga, gb, out, s); assert_close_entries(out.asnumpy(), O.mul(a, b), TOL, "mul")
    L.matrix_elementwise_add_by_const(ga, 1.5, out, s); assert_close_entries(out.asnumpy(), O.add_const(a, 1.5), TOL, "addc")
    L.matrix_elementwise_multiply_by_const(ga, -0.3, out, s); assert_close_entries(out.asnumpy(), O.mul_const(a, -0.3), TOL, "mulc")
    L.array_set(out, 2.25, s); np.testing.assert_array_equal(out.asnumpy(), O.array_set(shape, 2.25))
    L.relu(ga, out, s); np.testing.assert_array_equal(out.asnumpy(), O.relu(a).astype(np.float32))
    L.relu_gradient(ga, gb, out, s); np.testing.assert_array_equal(out.asnumpy(), O.relu_grad(a, b).astype(np.float32))
    flat = ts.empty((int(np.prod(shape)),))
    L.array_reshape(ga, flat, s); np.testing.assert_array_equal(flat.asnumpy(), a.ravel())


def test_elementwise_on_unaligned_views(ts, rng):
    # micro-tensor views start on arbitrary 4-byte boundaries: 5 rows of 3 floats split in 5
    a = rng.normal(size=(5, 3)).astype(np.float32)
    ga, out = ts.arr(a), ts.arr(np.zeros((5, 3), np.float32))
    ga.split_tensor(5); out.split_tensor(5)
    for i in range(5):
        ts.links.relu(ga.sTensor[i], out.sTensor[i], ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), np.maximum(a, 0))


def test_size_mismatch_is_rejected(ts):
    a, b = ts.empty((4,)), ts.empty((5,))
    with pytest.raises(RuntimeError):
        ts.links.relu(a, b)


@pytest.mark.parametrize("n", [5, 4096, 250001])
def test_optimizers(ts, n, rng):
    p0 = rng.normal(size=n).astype(np.float32)
    g = rng.normal(size=n).astype(np.float32)
    L, s = ts.links, ts.stream
    # SGD, 3 steps
    p, ref = ts.arr(p0), p0.copy()
    gg = ts.arr(g)
    for _ in range(3):
        L.sgd_update(p, gg, 0.1, s)
        ref = O.sgd_update(ref, g, 0.1).astype(np.float32)
    assert_close_entries(p.asnumpy(), ref, TOL, "sgd")
    for nesterov in (False, True):
        p, v = ts.arr(p0), ts.arr(np.zeros(n, np.float32))
        rp, rv = p0.copy(), np.zeros(n, np.float32)
        for _ in range(3):
            L.momentum_update(p, gg, v, 0.1, 0.9, nesterov, s)
            rp, rv = [t.astype(np.float32) for t in O.momentum_update(rp, g, rv, 0.1, 0.9, nesterov)]
        assert_close_entries(p.asnumpy(), rp, TOL, "momentum p"); assert_close_entries(v.asnumpy(), rv, TOL, "momentum v")
    p, acc = ts.arr(p0), ts.arr(np.zeros(n, np.float32))
    rp, racc = p0.copy(), np.zeros(n, np.float32)
    for _ in range(3):
        L.adagrad_update(p, gg, acc, 0.1, 1e-7, s)
        rp, racc = [t.astype(np.float32) for t in O.adagrad_update(rp, g, racc, 0.1, 1e-7)]
    assert_close_entries(p.asnumpy(), rp, TOL, "adagrad p"); assert_close_entries(acc.asnumpy(), racc, TOL, "adagrad acc")
    p, m, v = ts.arr(p0), ts.arr(np.zeros(n, np.float32)), ts.arr(np.zeros(n, np.float32))
    rp, rm, rv = p0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    b1t = b2t = 1.0
    for _ in range(3):
        b1t *= 0.9; b2t *= 0.999
        L.adam_update(p, gg, m, v, 0.01, 0.9, 0.999, b1t, b2t, 1e-7, s)
        rp, rm, rv = [t.astype(np.float32) for t in O.adam_update(rp, g, rm, rv, 0.01, 0.9, 0.999, b1t, b2t, 1e-7)]
    assert_close_entries(p.asnumpy(), rp, TOL, "adam p"); assert_close_entries(m.asnumpy(), rm, TOL, "adam m")
    assert_close_entries(v.asnumpy(), rv, TOL, "adam v")


# rows of at least 2048 columns in multiples of 4 take the block-per-row cross-entropy kernels
@pytest.mark.parametrize("rows,cols", [(128, 10), (64, 1000), (3, 1), (5, 4097), (300, 257), (9, 4096), (7, 32000),
                                       (5, 2050), (600, 2048)])
def test_softmax_and_cross_entropy(ts, rows, cols, rng):
    y = (rng.normal(size=(rows, cols)) * 3).astype(np.float32)
    lab = np.eye(cols, dtype=np.float32)[rng.randint(0, cols, rows)]
    gy, gl = ts.arr(y), ts.arr(lab)
    out = ts.empty((rows, cols))
    ts.links.softmax(gy, out, ts.stream)
    assert_close_entries(out.asnumpy(), O.softmax(y), TOL, "softmax")
    loss = ts.empty((1,))
    ts.links.softmax_cross_entropy(gy, gl, loss, ts.stream)
    assert_close_entries(loss.asnumpy(), O.softmax_ce(y, lab), TOL, "ce")
    g = ts.arr(np.array([1.7], np.float32))
    ts.links.softmax_cross_entropy_gradient(gy, gl, g, out, ts.stream)
    assert_close_entries(out.asnumpy(), O.softmax_ce_grad(y, lab, np.array([1.7], np.float32)), TOL, "ce grad")
    # smoothed (non one-hot) labels
    sm = (lab * 0.9 + 0.1 / cols).astype(np.float32)
    ts.links.softmax_cross_entropy(gy, ts.arr(sm), loss, ts.stream)
    assert_close_entries(loss.asnumpy(), O.softmax_ce(y, sm), TOL, "ce smoothed")


@pytest.mark.parametrize("cols", [1000, 4096])
def test_cross_entropy_uniform_logits_is_log_c(ts, cols):
    y = np.full((8, cols), -4.5, np.float32)
    lab = np.eye(cols, dtype=np.float32)[np.arange(8)]
    loss = ts.empty((1,))
    ts.links.softmax_cross_entropy(ts.arr(y), ts.arr(lab), loss, ts.stream)
    assert abs(loss.asnumpy()[0] - np.log(cols)) < 1e-4 * np.log(cols)


def test_cross_entropy_wide_rows_extreme_logits(ts, rng):
    """One dominant logit per row (the others underflow), in a 3-D tensor as the Transformer loss
    passes it: loss -> 0 where the label sits on it, gradient rows sum to zero."""
    y = (rng.normal(size=(2, 3, 4096)) * 2).astype(np.float32)
    hot = rng.randint(0, 4096, size=(2, 3))
    for a in range(2):
        for b in range(3):
            y[a, b, hot[a, b]] = 200.0
    lab = np.zeros_like(y)
    for a in range(2):
        for b in range(3):
            lab[a, b, hot[a, b]] = 1.0
    loss, out = ts.empty((1,)), ts.empty(y.shape)
    ts.links.softmax_cross_entropy(ts.arr(y), ts.arr(lab), loss, ts.stream)
    assert abs(float(loss.asnumpy()[0])) < 1e-3
    g = ts.arr(np.array([1.0], np.float32))
    ts.links.softmax_cross_entropy_gradient(ts.arr(y), ts.arr(lab), g, out, ts.stream)
    got = out.asnumpy()
    assert np.all(np.isfinite(got)) and np.abs(got.sum(axis=-1)).max() < 1e-5


# channels of at most 16384 values (N*H*W) take the one-pass kernels: 16, 32 or 64 values per thread
BN_SHAPES = [(4, 3, 5, 6), (2, 5, 7, 7), (16, 64, 56, 56), (8, 512, 14, 14), (3, 2, 1, 1), (64, 16, 32, 32),
             (64, 8, 14, 14), (32, 8, 17, 17), (20, 4, 20, 20), (64, 4, 16, 16), (64, 4, 16, 17), (17, 5, 16, 15)]


@pytest.mark.parametrize("shape", BN_SHAPES)
@pytest.mark.parametrize("saved", [False, True])
def test_batchnorm_forward_backward(ts, shape, saved, rng):
    C = shape[1]
    x = (rng.normal(size=shape) * 2 + rng.normal(size=(1, C, 1, 1)) * 3).astype(np.float32)
    gamma = rng.normal(size=(1, C, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, C, 1, 1)).astype(np.float32)
    dy = rng.normal(size=shape).astype(np.float32)
    eps = 0.01
    gx, gg, gb, gdy = ts.arr(x), ts.arr(gamma), ts.arr(beta), ts.arr(dy)
    y, dx = ts.empty(shape), ts.empty(shape)
    dg, db = ts.empty((1, C, 1, 1)), ts.empty((1, C, 1, 1))
    sm = ts.empty((1, C, 1, 1)) if saved else None
    sv = ts.empty((1, C, 1, 1)) if saved else None
    ts.links.CuDNN_Batch_Normalization(gx, gg, gb, y, sm, sv, 0.99, eps, ts.stream)
    ry, mean, var = O.batchnorm_forward(x, gamma, beta, eps)
    assert_close_entries(y.asnumpy(), ry, TOL, "bn fwd")
    if saved:
        assert_close_entries(sm.asnumpy().ravel(), mean, TOL, "saved mean")
        assert_close_entries(sv.asnumpy().ravel(), 1 / np.sqrt(var + eps), TOL, "saved inv-std")
    ts.links.CuDNN_Batch_Normalization_gradient(gdy, gx, gg, dx, dg, db, sm, sv, eps, ts.stream)
    rdx, rdg, rdb = O.batchnorm_backward(dy, x, gamma, eps)
    assert_close_entries(dx.asnumpy(), rdx, TOL, "bn dx")
    assert_close_entries(dg.asnumpy().ravel(), rdg, TOL, "bn dgamma")
    assert_close_entries(db.asnumpy().ravel(), rdb, TOL, "bn dbeta")


def test_batchnorm_on_micro_tensor_views_differs_from_full_batch(ts, rng):
    """BN over a micro-batch is BN of that micro-batch (not of the full batch): each view
    must match the oracle on its own rows."""
    x = rng.normal(size=(8, 4, 6, 6)).astype(np.float32)
    gamma, beta = np.ones((1, 4, 1, 1), np.float32), np.zeros((1, 4, 1, 1), np.float32)
    gx, y = ts.arr(x), ts.empty(x.shape)
    gx.split_tensor(4); y.split_tensor(4)
    gg, gb = ts.arr(gamma), ts.arr(beta)
    for i in range(4):
        ts.links.CuDNN_Batch_Normalization(gx.sTensor[i], gg, gb, y.sTensor[i], None, None, 0.99, 0.01, ts.stream)
    got = y.asnumpy()
    for i in range(4):
        assert_close(got[2 * i:2 * i + 2], O.batchnorm_forward(x[2 * i:2 * i + 2], gamma, beta, 0.01)[0], TOL, "micro bn")


POOL_CASES = [
    # shape, kH, kW, pad, stride
    ((2, 3, 8, 8), 2, 2, 0, 2),          # vectorised 2x2 path
    ((4, 64, 56, 56), 2, 2, 0, 2),
    ((2, 3, 14, 14), 2, 2, 0, 2),        # W % 4 != 0 -> generic path
    ((2, 3, 7, 7), 3, 3, 1, 2),          # ResNet pool (exact)
    ((2, 3, 8, 8), 3, 3, 1, 2),          # floors
    ((2, 2, 9, 11), 3, 3, 0, 2),         # Inception pool
    ((1, 2, 6, 7), 2, 3, 0, 1),          # overlapping, non-square
    ((2, 3, 9, 10), 3, 3, 1, 1),         # 3x3 stride 1: nine windows over an element
    ((2, 3, 9, 10), 2, 2, 0, 1),         # 2x2 stride 1
    ((2, 3, 9, 10), 2, 2, 1, 2),         # 2x2 stride 2 with padding
    ((1, 2, 12, 12), 3, 3, 0, 3),        # 3x3 stride 3: disjoint windows
    ((1, 2, 11, 9), 2, 2, 0, 3),         # gaps between windows
    ((4, 16, 57, 57), 3, 3, 1, 2),       # larger overlapping case
]


@pytest.mark.parametrize("shape,kH,kW,pad,stride", POOL_CASES)
@pytest.mark.parametrize("ties", [False, True])
@pytest.mark.parametrize("family", ["plain", "cudnn"])
def test_maxpool_bit_exact(ts, shape, kH, kW, pad, stride, ties, family, rng):
    if ties:
        x = rng.randint(0, 3, size=shape).astype(np.float32)     # many equal values per window
    else:
        x = rng.normal(size=shape).astype(np.float32)
    ref = O.max_pool(x, kH, kW, pad, stride)
    dy = rng.normal(size=ref.shape).astype(np.float32)
    gx, gdy = ts.arr(x), ts.arr(dy)
    y, dx = ts.empty(ref.shape), ts.empty(shape)
    if family == "plain":
        ts.links.max_pooling2d(gx, kH, kW, y, pad, stride, ts.stream)
        ts.links.max_pooling2d_gradient(gx, gdy, kH, kW, dx, pad, stride, ts.stream)
    else:
        ts.links.CuDNN_max_pooling2d(gx, kH, kW, y, pad, stride, ts.stream)
        ts.links.CuDNN_max_pooling2d_gradient(y, gdy, gx, kH, kW, dx, pad, stride, ts.stream)
    np.testing.assert_array_equal(y.asnumpy(), ref)
    got_dx = dx.asnumpy()
    ref_dx = O.max_pool_grad(x, dy, kH, kW, pad, stride, dtype=np.float32)   # fp32 accumulation, window order
    np.testing.assert_array_equal(got_dx, ref_dx)
    # the argmax positions themselves: route a gradient of distinct powers of two... use index-valued dy
    if not (stride < max(kH, kW)):       # non-overlapping windows: dx != 0 exactly at the argmax
        arg = O.max_pool_argmax(x, kH, kW, pad, stride)
        idy = (np.arange(ref.size, dtype=np.float32).reshape(ref.shape) + 1)
        ts.links.max_pooling2d_gradient(gx, ts.arr(idy), kH, kW, dx, pad, stride, ts.stream)
        got = dx.asnumpy().reshape(shape[0], shape[1], -1)
        pos = np.take_along_axis(got, arg.reshape(shape[0], shape[1], -1), axis=2).reshape(ref.shape)
        np.testing.assert_array_equal(pos, idy)


def test_concat_slice_bit_exact(ts, rng):
    for sa, sb, axis in [((2, 3, 4, 4), (2, 5, 4, 4), 1), ((3, 4), (2, 4), 0), ((2, 3, 5), (2, 3, 2), 2),
                         ((32, 96, 35, 35), (32, 96, 35, 35), 1)]:
        a = rng.normal(size=sa).astype(np.float32)
        b = rng.normal(size=sb).astype(np.float32)
        ref = O.concat(a, b, axis)
        out = ts.empty(ref.shape)
        ts.links.concat(ts.arr(a), ts.arr(b), out, axis, ts.stream)
        np.testing.assert_array_equal(out.asnumpy(), ref)
        ga, gb = ts.empty(sa), ts.empty(sb)
        ts.links.concat_gradient(out, ga, axis, 0, ts.stream)
        ts.links.concat_gradient(out, gb, axis, 1, ts.stream)
        np.testing.assert_array_equal(ga.asnumpy(), O.concat_grad(ref, sa, axis, 0))
        np.testing.assert_array_equal(gb.asnumpy(), O.concat_grad(ref, sb, axis, 1))
    x = rng.normal(size=(4, 6, 5, 7)).astype(np.float32)
    begin, oshape = (1, 2, 0, 3), (2, 3, 5, 2)
    out = ts.empty(oshape)
    ts.links.matrix_slice(ts.arr(x), out, begin, ts.stream)
    np.testing.assert_array_equal(out.asnumpy(), O.slice_(x, begin, oshape))
    back = ts.empty(x.shape)
    ts.links.matrix_slice_gradient(out, back, begin, ts.stream)
    np.testing.assert_array_equal(back.asnumpy(), O.slice_grad(out.asnumpy(), begin, x.shape))


def test_batch_split_views_are_zero_copy_and_exact(ts, rng):
    x = rng.normal(size=(10, 3, 4, 4)).astype(np.float32)
    gx = ts.arr(x)
    gx.split_tensor(4)
    assert [t.shape for t in gx.sTensor] == O.split_shape(x.shape, 4)
    for i, t in enumerate(gx.sTensor):
        off, shp = O.micro_tensor_view(x.shape, 4, i)
        assert t.data_ptr == gx.data_ptr + 4 * off
        np.testing.assert_array_equal(t.asnumpy(), x.ravel()[off:off + int(np.prod(shp))].reshape(shp))
    # per-sample op on the 4 micro-tensors == the op on the whole batch, bit for bit
    whole, parts = ts.empty(x.shape), ts.empty(x.shape)
    ts.links.relu(gx, whole, ts.stream)
    parts.split_tensor(4)
    for i in range(4):
        ts.links.relu(gx.sTensor[i], parts.sTensor[i], ts.stream)
    np.testing.assert_array_equal(whole.asnumpy(), parts.asnumpy())


def test_pool_and_profiler_and_events(ts, rng):
    from tsplit_amd import gpu_memory_manager as mm, profiler, stream
    before = mm.get_gpu_memory()["used_size"].value
    a = ts.empty((1024, 1024))
    assert mm.get_gpu_memory()["used_size"].value - before == 4 << 20
    assert mm.judge_malloc((1024, 1024)) == 1
    assert mm.judge_malloc((1 << 20, 1 << 20)) == 0       # 4 TiB can never fit
    a.delete_itself()
    assert mm.get_gpu_memory()["used_size"].value == before
    a.malloc_itself()
    p = profiler.CreateProfiler()
    x = ts.arr(rng.normal(size=(256, 1024)))
    ts.links.relu(x, a if a.shape == x.shape else ts.empty(x.shape), None, p)
    assert p.time > 0 and abs(p.input_memory - 1.0) < 1e-6 and abs(p.output_memory - 1.0) < 1e-6
    ev = stream.create_event_handle(ts.ctx)
    ev.record(ts.stream); ev.sync()
    assert ev.query() is True
    # async copies with a pinned host array
    host = ts.nd.array(rng.normal(size=(64, 64)).astype(np.float32), ts.nd.cpu(0))
    dev = ts.empty((64, 64))
    dev.async_h2d(host, ts.stream, dev.cpu2gpu_event)
    dev.cpu2gpu_event.sync()
    back = ts.nd.empty((64, 64), ts.nd.cpu(0))
    back.async_d2h(dev, ts.stream, dev.gpu2cpu_event)
    dev.gpu2cpu_event.sync()
    np.testing.assert_array_equal(back.asnumpy(), host.asnumpy())


@pytest.mark.parametrize("shape", [(4, 8, 6, 6), (3, 5, 7, 9), (16, 64, 56, 56)])
def test_fused_batchnorm_relu_equals_the_two_call_sequence(ts, shape, rng):
    """The fused symbols have no counterpart in the reference; their contract is to reproduce
    BatchNorm followed by Relu (and the reverse sweep) exactly, and through them the oracle."""
    C = shape[1]
    x = rng.normal(size=shape).astype(np.float32)
    gamma = (1 + 0.1 * rng.normal(size=(1, C, 1, 1))).astype(np.float32)
    beta = (0.1 * rng.normal(size=(1, C, 1, 1))).astype(np.float32)
    dy = rng.normal(size=shape).astype(np.float32)
    L, s = ts.links, ts.stream
    gx, gg, gb, gdy = ts.arr(x), ts.arr(gamma), ts.arr(beta), ts.arr(dy)
    # two calls per direction
    sm, sv = ts.empty((1, C, 1, 1)), ts.empty((1, C, 1, 1))
    y_bn, y = ts.empty(shape), ts.empty(shape)
    L.CuDNN_Batch_Normalization(gx, gg, gb, y_bn, sm, sv, 0.99, 0.01, s)
    L.relu(y_bn, y, s)
    d_bn, dx, dg, db = ts.empty(shape), ts.empty(shape), ts.empty((1, C, 1, 1)), ts.empty((1, C, 1, 1))
    L.relu_gradient(y_bn, gdy, d_bn, s)
    L.CuDNN_Batch_Normalization_gradient(d_bn, gx, gg, dx, dg, db, sm, sv, 0.01, s)
    # one call per direction
    fm, fv = ts.empty((1, C, 1, 1)), ts.empty((1, C, 1, 1))
    fy, fdx, fdg, fdb = ts.empty(shape), ts.empty(shape), ts.empty((1, C, 1, 1)), ts.empty((1, C, 1, 1))
    L.batch_norm_relu(gx, gg, gb, fy, fm, fv, 0.01, s)
    L.batch_norm_relu_gradient(gdy, gx, gg, gb, fdx, fdg, fdb, fm, fv, 0.01, s)
    ref_y = O.relu(O.batchnorm_forward(x, gamma, beta, 0.01)[0])
    assert_close(fy.asnumpy(), ref_y, TOL, "bn+relu")
    assert_close(fy.asnumpy(), y.asnumpy(), 1e-6, "fused vs two calls, forward")
    # the Relu gate is discontinuous at 0: compare where the pre-activation is clearly off zero
    z = O.batchnorm_forward(x, gamma, beta, 0.01)[0]
    g = O.relu_grad(z, dy)
    rdx, rdg, rdb = O.batchnorm_backward(g, x, gamma, 0.01)
    assert_close(fdx.asnumpy(), rdx, 5e-4, "bn+relu dx")
    assert_close(fdg.asnumpy().ravel(), rdg.ravel(), 5e-4, "bn+relu dgamma")
    assert_close(fdb.asnumpy().ravel(), rdb.ravel(), 5e-4, "bn+relu dbeta")
    assert_close(fdx.asnumpy(), dx.asnumpy(), 5e-4, "fused vs two calls, dx")
    np.testing.assert_allclose(fm.asnumpy(), sm.asnumpy(), rtol=1e-6)


def test_fused_batchnorm_relu_needs_saved_statistics(ts):
    x, g, b, y = ts.empty((2, 3, 4, 4)), ts.empty((1, 3, 1, 1)), ts.empty((1, 3, 1, 1)), ts.empty((2, 3, 4, 4))
    with pytest.raises(Exception):
        ts.links.batch_norm_relu(x, g, b, y, None, None, 0.01, ts.stream)


@pytest.mark.parametrize("kind", ["sgd", "momentum", "nesterov"])
def test_optimizer_update_of_many_parameters_in_one_launch(ts, kind, rng):
    """TSplit_OptimizerUpdateMulti against the per-parameter symbols (same bits) and the oracle, three
    steps over parameters of awkward sizes: single values, tails of 1 - 3 elements, an array longer than
    one block's share, a view that starts off a 16-byte boundary, an empty array."""
    L, s = ts.links, ts.stream
    shapes = [(1,), (3,), (5,), (1023,), (4096,), (4097,), (64, 3, 3, 3), (1, 512, 1, 1), (100003,), (300, 257)]
    ps = [rng.normal(size=sh).astype(np.float32) for sh in shapes]
    one, many = [ts.arr(p) for p in ps], [ts.arr(p) for p in ps]
    vel_one, vel_many = [ts.arr(np.zeros_like(p)) for p in ps], [ts.arr(np.zeros_like(p)) for p in ps]
    # an unaligned view: rows 1.. of a 5 x 3 array start 12 bytes into it
    base_one, base_many = ts.arr(rng.normal(size=(5, 3))), None
    base_many = ts.arr(base_one.asnumpy())
    vb_one, vb_many = ts.arr(np.zeros((5, 3))), ts.arr(np.zeros((5, 3)))
    for b in (base_one, base_many, vb_one, vb_many):
        b.split_tensor(5)
    views = lambda arr: [arr.sTensor[1], arr.sTensor[3]]
    ref_p = [p.astype(np.float64) for p in ps] + [base_one.asnumpy()[1:2].astype(np.float64), base_one.asnumpy()[3:4].astype(np.float64)]
    ref_v = [np.zeros_like(p) for p in ref_p]
    lr, mom = 0.05, 0.9
    for step in range(3):
        gs = [rng.normal(size=p.shape).astype(np.float32) for p in ref_p]
        g_dev = [ts.arr(g) for g in gs]
        p_one, p_many = one + views(base_one), many + views(base_many)
        v_one, v_many = vel_one + views(vb_one), vel_many + views(vb_many)
        for p, g, v in zip(p_one, g_dev, v_one):
            if kind == "sgd":
                L.sgd_update(p, g, lr, s)
            else:
                L.momentum_update(p, g, v, lr, mom, kind == "nesterov", s)
        L.optimizer_update_multi(p_many, g_dev, None if kind == "sgd" else v_many, lr, mom, kind == "nesterov", s)
        for i, g in enumerate(gs):
            if kind == "sgd":
                ref_p[i] = O.sgd_update(ref_p[i], g, lr)
            else:
                ref_p[i], ref_v[i] = O.momentum_update(ref_p[i], g, ref_v[i], lr, mom, kind == "nesterov")
    for a, b, r in zip(one + views(base_one), many + views(base_many), ref_p):
        np.testing.assert_array_equal(b.asnumpy(), a.asnumpy())
        assert_close(b.asnumpy(), r, TOL, "parameter after three updates")
    for a, b in zip(vel_one, vel_many):
        np.testing.assert_array_equal(b.asnumpy(), a.asnumpy())
    # the rows of the 5 x 3 arrays that were not listed are untouched
    np.testing.assert_array_equal(base_many.asnumpy()[[0, 2, 4]], base_one.asnumpy()[[0, 2, 4]])
    L.optimizer_update_multi([], [], None, lr, stream=s)         # nothing to do


def test_optimizer_update_of_many_parameters_survives_stream_destruction(ts, rng):
    """The list of arrays a stream last updated is remembered so that it is uploaded once.  A stream
    that is destroyed takes its device copy with it: a new stream updating the very same arrays
    uploads the list again (streams are created and destroyed several times so that a handle value
    is likely to come back), and a changed list on a live stream is uploaded too."""
    from tsplit_amd import stream as S
    L = ts.links
    shapes = [(7,), (4096,), (64, 3, 3, 3), (100003,)]
    ps = [rng.normal(size=sh).astype(np.float32) for sh in shapes]
    one, many = [ts.arr(p) for p in ps], [ts.arr(p) for p in ps]
    v_one, v_many = [ts.arr(np.zeros_like(p)) for p in ps], [ts.arr(np.zeros_like(p)) for p in ps]
    lr, mom = 0.05, 0.9
    for round_ in range(4):
        s = S.create_stream_handle(ts.ctx)
        gs = [ts.arr(rng.normal(size=sh)) for sh in shapes]
        for p, g, v in zip(one, gs, v_one):
            L.momentum_update(p, g, v, lr, mom, False, s)
        L.optimizer_update_multi(many, gs, v_many, lr, mom, False, s)
        # a shorter list on the same stream, then the full one again
        L.momentum_update(one[1], gs[1], v_one[1], lr, mom, False, s)
        L.optimizer_update_multi(many[1:2], gs[1:2], v_many[1:2], lr, mom, False, s)
        for p, g, v in zip(one, gs, v_one):
            L.momentum_update(p, g, v, lr, mom, False, s)
        L.optimizer_update_multi(many, gs, v_many, lr, mom, False, s)
        s.sync()
        for a, b in zip(one + v_one, many + v_many):
            np.testing.assert_array_equal(b.asnumpy(), a.asnumpy())
        del s       # DLStreamDestroy
