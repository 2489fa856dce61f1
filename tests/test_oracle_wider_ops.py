"""Pins the oracle functions of the operators around the core path (average pooling,
broadcast/reduce, pad, batched matmul, transpose, one-hot, where, embedding, elementwise
math) against literal loops, library routines and identities."""
import numpy as np
import pytest

from oracle import loops, ops

POOL_CASES = [
    # N, C, H, W, kH, kW, pad, stride
    (2, 3, 7, 7, 7, 7, 0, 7),     # ResNet global pool
    (1, 2, 8, 8, 8, 8, 0, 1),     # Inception global pool
    (2, 2, 6, 5, 3, 3, 1, 1),     # Inception 3x3 same pool: clipped windows keep divisor 9
    (1, 2, 7, 7, 3, 3, 1, 2),
    (1, 1, 6, 6, 2, 2, 0, 2),
    (1, 2, 8, 8, 3, 3, 1, 2),     # floors
]


@pytest.mark.parametrize("case", POOL_CASES)
def test_avg_pool_matches_loops(case, rng):
    N, C, H, W, kH, kW, pad, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    y = ops.avg_pool(x, kH, kW, pad, s)
    np.testing.assert_allclose(y, loops.avg_pool_loops(x.astype(np.float64), kH, kW, pad, s), rtol=1e-13, atol=1e-13)
    dy = rng.normal(size=y.shape).astype(np.float32)
    dx = ops.avg_pool_grad(dy, x.shape, kH, kW, pad, s)
    np.testing.assert_allclose(dx, loops.avg_pool_grad_loops(dy.astype(np.float64), x.shape, kH, kW, pad, s),
                               rtol=1e-13, atol=1e-13)
    # adjoint identity <P x, dy> == <x, P^T dy>
    np.testing.assert_allclose(np.sum(y * dy), np.sum(x.astype(np.float64) * dx), rtol=1e-10)


def test_avg_pool_is_depthwise_correlation_with_constant_filter(rng):
    x = rng.normal(size=(2, 3, 6, 6)).astype(np.float32)
    y = ops.avg_pool(x, 3, 3, 1, 1)
    for c in range(3):
        w = np.full((1, 1, 3, 3), 1.0 / 9.0, np.float64)
        yc = ops.conv2d(x[:, c:c + 1], w.astype(np.float32), 1, 1, 1)
        np.testing.assert_allclose(y[:, c:c + 1], yc, rtol=1e-6)
    # a constant image: interior 1, corners 4/9, edges 6/9
    y1 = ops.avg_pool(np.ones((1, 1, 4, 4), np.float32), 3, 3, 1, 1)[0, 0]
    assert y1[1, 1] == 1.0 and abs(y1[0, 0] - 4 / 9) < 1e-15 and abs(y1[0, 1] - 6 / 9) < 1e-15


def test_broadcast_and_axis_zero_reduce(rng):
    b = rng.normal(size=(5,)).astype(np.float32)
    np.testing.assert_array_equal(ops.broadcast_to(b, (4, 5)), loops.broadcast_flat_loops(b.astype(np.float64), (4, 5)))
    m = rng.normal(size=(3, 5)).astype(np.float32)
    np.testing.assert_array_equal(ops.broadcast_to(m, (2, 3, 5)), loops.broadcast_flat_loops(m.astype(np.float64), (2, 3, 5)))
    x = rng.normal(size=(7, 3, 5)).astype(np.float32)
    r = ops.reduce_sum_axis_zero(x)
    ref = np.zeros((3, 5))
    for i in range(7):
        ref += x[i].astype(np.float64)
    np.testing.assert_allclose(r, ref, rtol=1e-14)
    # adjoint pair: <broadcast(b), x> == <b, reduce(x)>
    v = rng.normal(size=(3, 5)).astype(np.float32)
    np.testing.assert_allclose(np.sum(ops.broadcast_to(v, x.shape) * x), np.sum(v.astype(np.float64) * r), rtol=1e-10)


def test_conv_bias_broadcast_and_reduce(rng):
    b = rng.normal(size=(3,)).astype(np.float32)
    out = ops.conv2d_broadcast_to(b, (2, 3, 4, 5))
    for n in range(2):
        for c in range(3):
            assert np.all(out[n, c] == np.float64(b[c]))
    x = rng.normal(size=(2, 3, 4, 5)).astype(np.float32)
    r = ops.conv2d_reduce_sum(x)
    for c in range(3):
        s = 0.0
        for n in range(2):
            for h in range(4):
                for w in range(5):
                    s += float(x[n, c, h, w])
        assert abs(r[c] - s) < 1e-12
    np.testing.assert_allclose(np.sum(out * x), np.sum(b.astype(np.float64) * r), rtol=1e-10)


@pytest.mark.parametrize("in_shape,out_shape,add_axes", [
    ((4, 4), (2, 3, 4, 4), None),            # causal mask of the transformer
    ((3, 1, 4), (2, 3, 5, 4), None),
    ((2, 4), (2, 3, 4), [1]),
    ((3,), (2, 3, 4), [0, 2]),
    ((2, 3), (2, 5, 3, 4), [1, 3]),
])
def test_broadcast_shape_matches_index_walk(in_shape, out_shape, add_axes, rng):
    x = rng.normal(size=in_shape).astype(np.float32)
    np.testing.assert_array_equal(ops.broadcast_shape(x, out_shape, add_axes),
                                  loops.broadcast_shape_loops(x.astype(np.float64), out_shape, add_axes))


def test_reduce_sum_axes(rng):
    x = rng.normal(size=(3, 4, 5, 2)).astype(np.float32)
    for axes in ([0], [3], [1, 2], [0, 1], [0, 2, 3], [0, 1, 2, 3]):
        r = ops.reduce_sum(x, axes)
        kept = [d for d in range(4) if d not in axes]
        ref = np.zeros([x.shape[d] for d in kept])
        for idx in np.ndindex(*x.shape):
            ref[tuple(idx[d] for d in kept)] += float(x[idx])
        np.testing.assert_allclose(r, ref, rtol=1e-12, atol=1e-12)
        assert ops.reduce_sum(x, axes, keepdims=True).shape == tuple(1 if d in axes else x.shape[d] for d in range(4))


@pytest.mark.parametrize("paddings", [[(1, 1), (1, 1)], [(0, 2), (3, 0)], [(1, 0), (0, 0), (2, 1)],
                                       [(1, 1), (0, 1), (1, 0), (2, 2)]])
def test_pad_and_gradient(paddings, rng):
    x = rng.normal(size=(2, 3, 4, 5)).astype(np.float32)
    y = ops.pad(x, paddings, 0.5)
    np.testing.assert_array_equal(y, loops.pad_loops(x.astype(np.float64), paddings, 0.5))
    np.testing.assert_array_equal(ops.pad_grad(y, paddings), x.astype(np.float64))      # crop undoes pad
    dy = rng.normal(size=y.shape).astype(np.float32)
    np.testing.assert_allclose(np.sum(ops.pad(x, paddings, 0.0) * dy), np.sum(x * ops.pad_grad(dy, paddings)), rtol=1e-10)


@pytest.mark.parametrize("tA,tB", [(False, False), (True, False), (False, True), (True, True)])
def test_batch_matmul(tA, tB, rng):
    a_shape = (2, 3, 5, 4) if tA else (2, 3, 4, 5)
    b_shape = (2, 3, 6, 5) if tB else (2, 3, 5, 6)
    A = rng.normal(size=a_shape).astype(np.float32)
    B = rng.normal(size=b_shape).astype(np.float32)
    C = ops.batch_matmul(A, tA, B, tB)
    assert C.shape == (2, 3, 4, 6)
    np.testing.assert_allclose(C, loops.batch_matmul_loops(A, tA, B, tB), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape,perm", [((3, 5), (1, 0)), ((2, 3, 4, 5), (0, 2, 1, 3)), ((2, 3, 4), (2, 0, 1)),
                                        ((2, 3, 4, 5), (3, 2, 1, 0)), ((2, 3, 4), (0, 1, 2))])
def test_transpose(shape, perm, rng):
    x = rng.normal(size=shape).astype(np.float32)
    y = ops.transpose(x, perm)
    np.testing.assert_array_equal(y, loops.transpose_loops(x, perm))
    inv = np.argsort(perm)
    np.testing.assert_array_equal(ops.transpose(y, inv), x)


def test_one_hot_where_embedding(rng):
    ids = rng.randint(0, 7, size=(3, 4)).astype(np.float32)
    oh = ops.one_hot(ids, 7)
    np.testing.assert_array_equal(oh, loops.one_hot_loops(ids, 7))
    assert np.all(oh.sum(-1) == 1) and np.all(oh.argmax(-1) == ids)
    assert ops.one_hot(np.array([9.0, 2.5], np.float32), 4).sum() == 0       # out of range / non-integer ids match nothing
    c = (rng.rand(3, 4) > 0.5).astype(np.float32)
    a, b = rng.normal(size=(3, 4)).astype(np.float32), rng.normal(size=(3, 4)).astype(np.float32)
    w = ops.where(c, a, b)
    for i in np.ndindex(3, 4):
        assert w[i] == (a[i] if c[i] else b[i])
    table = rng.normal(size=(7, 5)).astype(np.float32)
    e = ops.embedding_lookup(table, ids)
    np.testing.assert_array_equal(e, loops.embedding_loops(table, ids))
    np.testing.assert_array_equal(e, np.einsum("...v,vd->...d", oh, table))   # lookup == one-hot matmul
    dy = rng.normal(size=e.shape).astype(np.float32)
    g = ops.embedding_lookup_grad(dy, ids, table.shape)
    np.testing.assert_allclose(g, loops.embedding_grad_loops(dy, ids, table.shape), rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(g, np.einsum("abv,abd->vd", oh.astype(np.float64), dy.astype(np.float64)), rtol=1e-12, atol=1e-12)


def test_elementwise_math_identities(rng):
    x = (rng.rand(50) * 4 + 0.1).astype(np.float32)
    xd = x.astype(np.float64)
    np.testing.assert_allclose(ops.sqrt(x) ** 2, xd, rtol=1e-14)
    np.testing.assert_allclose(ops.rsqrt(x) * ops.sqrt(x), 1.0, rtol=1e-14)
    z = rng.normal(size=50).astype(np.float32)
    zd = z.astype(np.float64)
    s = ops.sigmoid(z)
    np.testing.assert_allclose(np.log(s / (1 - s)), zd, rtol=1e-10, atol=1e-12)           # logit inverts it
    np.testing.assert_allclose(s, 1.0 / (1.0 + 1.0 / np.exp(zd)), rtol=1e-14)            # the CUDA form, src/ops/Sigmoid.cu:6
    np.testing.assert_allclose(np.arctanh(ops.tanh(z)), zd, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(ops.tanh(z), 2 * ops.sigmoid(2 * z) - 1, rtol=1e-12, atol=1e-14)
    np.testing.assert_array_equal(ops.opposite(z), -zd)
    np.testing.assert_allclose(ops.div_const(3.0, x) * xd, 3.0, rtol=1e-14)              # constant over tensor
    np.testing.assert_allclose(ops.divide(z, x) * xd, zd, rtol=1e-14)
