"""Seeded sweeps of random shapes against the CPU oracle for the operators whose kernels are chosen
by shape: matrix products (all transpose forms; tile family, split-K, ragged tiles and a ragged
last k-step), batched products, and max / average pooling (window, padding and stride drawn at
random; max pooling bit-exact including tie order, through both symbol families)."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu


def _dims(rng, hi):
    pool = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 513]
    return int(rng.choice([d for d in pool if d <= hi]))


def _matmul_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        M, N = _dims(rng, 513), _dims(rng, 513)
        K = int(rng.choice([1, 3, 4, 15, 16, 17, 20, 32, 48, 63, 64, 100, 256, 1000, 4099]))
        out.append((M, N, K, bool(rng.randint(2)), bool(rng.randint(2))))
    return out


@pytest.mark.parametrize("M,N,K,tA,tB", _matmul_cases(7, 200))
def test_random_matmul(M, N, K, tA, tB):
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((M * 131 + N * 17 + K) % (2 ** 31))
    A = rng.normal(size=(K, M) if tA else (M, K)).astype(np.float32)
    B = rng.normal(size=(N, K) if tB else (K, N)).astype(np.float32)
    C = ndarray.empty((M, N), ctx)
    gpu_links.matrix_multiply(ndarray.array(A, ctx), tA, ndarray.array(B, ctx), tB, C)
    err = assert_close(C.asnumpy(), O.matmul(A, tA, B, tB), 2e-3, f"matmul {M}x{N}x{K} tA={tA} tB={tB}")
    assert err < 1e-4


def _batched_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        lead = tuple(int(v) for v in rng.randint(1, 5, size=rng.randint(1, 3)))
        out.append((lead, _dims(rng, 300), _dims(rng, 300), int(rng.choice([1, 5, 16, 17, 33, 64, 100, 130])),
                    bool(rng.randint(2)), bool(rng.randint(2))))
    return out


@pytest.mark.parametrize("lead,M,N,K,tA,tB", _batched_cases(11, 80))
def test_random_batched_matmul(lead, M, N, K, tA, tB):
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((M * 131 + N * 17 + K + len(lead)) % (2 ** 31))
    A = rng.normal(size=lead + ((K, M) if tA else (M, K))).astype(np.float32)
    B = rng.normal(size=lead + ((N, K) if tB else (K, N))).astype(np.float32)
    C = ndarray.empty(lead + (M, N), ctx)
    gpu_links.batch_matrix_multiply(ndarray.array(A, ctx), tA, ndarray.array(B, ctx), tB, C)
    err = assert_close(C.asnumpy(), O.batch_matmul(A, tA, B, tB), 2e-3, f"batched {lead} {M}x{N}x{K} tA={tA} tB={tB}")
    assert err < 1e-4


def _pool_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        kH = int(rng.choice([1, 2, 3, 4, 5]))
        kW = kH if rng.rand() < 0.7 else int(rng.choice([1, 2, 3, 4, 5]))
        stride = int(rng.choice([1, 2, 2, 3]))
        pad = int(rng.randint(0, min(kH, kW) // 2 + 1))          # padding stays below the window
        H, W = int(rng.randint(1, 40)), int(rng.randint(1, 40))
        if H + 2 * pad < kH or W + 2 * pad < kW:
            continue
        out.append(((int(rng.choice([1, 2, 3])), int(rng.choice([1, 3, 16, 33])), H, W), kH, kW, pad, stride))
    return out


@pytest.mark.parametrize("shape,kH,kW,pad,stride", _pool_cases(3, 150))
def test_random_pooling(shape, kH, kW, pad, stride):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((shape[2] * 41 + shape[3] * 7 + kH * 3 + kW + stride) % (2 ** 31))
    ties = rng.rand() < 0.4
    x = (rng.randint(0, 3, size=shape) if ties else rng.normal(size=shape)).astype(np.float32)
    ref = O.max_pool(x, kH, kW, pad, stride)
    dy = rng.normal(size=ref.shape).astype(np.float32)
    gx, gdy = ndarray.array(x, ctx), ndarray.array(dy, ctx)
    y, dx = ndarray.empty(ref.shape, ctx), ndarray.empty(shape, ctx)
    ref_dx = O.max_pool_grad(x, dy, kH, kW, pad, stride, dtype=np.float32)
    L.max_pooling2d(gx, kH, kW, y, pad, stride)
    L.max_pooling2d_gradient(gx, gdy, kH, kW, dx, pad, stride)
    np.testing.assert_array_equal(y.asnumpy(), ref)
    np.testing.assert_array_equal(dx.asnumpy(), ref_dx)
    L.CuDNN_max_pooling2d(gx, kH, kW, y, pad, stride)
    L.CuDNN_max_pooling2d_gradient(y, gdy, gx, kH, kW, dx, pad, stride)
    np.testing.assert_array_equal(y.asnumpy(), ref)
    np.testing.assert_array_equal(dx.asnumpy(), ref_dx)
    # average pooling on the same geometry
    L.average_pooling2d(gx, kH, kW, y, pad, stride)
    L.average_pooling2d_gradient(gdy, kH, kW, dx, pad, stride)
    assert_close(y.asnumpy(), O.avg_pool(x, kH, kW, pad, stride), 1e-4, "avg_pool")
    assert_close(dx.asnumpy(), O.avg_pool_grad(dy, shape, kH, kW, pad, stride), 1e-4, "avg_pool_grad")


def _bn_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        N, C = int(rng.choice([1, 2, 3, 8, 32])), int(rng.choice([1, 3, 16, 33, 64, 130]))
        H, W = int(rng.randint(1, 40)), int(rng.randint(1, 40))
        if rng.rand() < 0.25:
            H, W = int(rng.choice([56, 64, 75])), int(rng.choice([56, 64, 75]))     # beyond one pass per channel
        if N * C * H * W > 3e6:
            N = 1
        out.append(((N, C, H, W), bool(rng.randint(2))))
    return out


@pytest.mark.parametrize("shape,saved", _bn_cases(5, 80))
def test_random_batchnorm(shape, saved):
    """Plain and fused BatchNorm(+Relu), forward and gradient, with and without saved statistics."""
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    C = shape[1]
    rng = np.random.RandomState((shape[0] * 7 + C * 131 + shape[2] * 31 + shape[3]) % (2 ** 31))
    x = (rng.normal(size=shape) * 2 + rng.normal(size=(1, C, 1, 1)) * 3).astype(np.float32)
    gamma = rng.normal(size=(1, C, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, C, 1, 1)).astype(np.float32)
    dy = rng.normal(size=shape).astype(np.float32)
    eps = 0.01
    arr = lambda a: ndarray.array(a, ctx)
    gx, gg, gb, gdy = arr(x), arr(gamma), arr(beta), arr(dy)
    y, dx = ndarray.empty(shape, ctx), ndarray.empty(shape, ctx)
    dg, db = ndarray.empty((1, C, 1, 1), ctx), ndarray.empty((1, C, 1, 1), ctx)
    sm, sv = ndarray.empty((1, C, 1, 1), ctx), ndarray.empty((1, C, 1, 1), ctx)
    L.CuDNN_Batch_Normalization(gx, gg, gb, y, sm if saved else None, sv if saved else None, 0.99, eps)
    ry, mean, var = O.batchnorm_forward(x, gamma, beta, eps)
    assert_close(y.asnumpy(), ry, 1e-4, "bn fwd")
    L.CuDNN_Batch_Normalization_gradient(gdy, gx, gg, dx, dg, db, sm if saved else None, sv if saved else None, eps)
    rdx, rdg, rdb = O.batchnorm_backward(dy, x, gamma, eps)
    assert_close(dx.asnumpy(), rdx, 1e-4, "bn dx")
    assert_close(dg.asnumpy().ravel(), rdg, 1e-4, "bn dgamma")
    assert_close(db.asnumpy().ravel(), rdb, 1e-4, "bn dbeta")
    # fused with Relu: max(BN(x), 0) and the reference's Relu derivative (1/2 at zero) in front of the BN gradient
    L.batch_norm_relu(gx, gg, gb, y, sm, sv, eps)
    fused_y = y.asnumpy()
    assert_close(fused_y, np.maximum(ry, 0), 1e-4, "bn+relu fwd")
    L.batch_norm_relu_gradient(gdy, gx, gg, gb, dx, dg, db, sm, sv, eps)
    # the gate follows the sign fp32 arithmetic gave z = BN(x) (a z within rounding of zero may have
    # the other sign in float64; exact zeros, where the derivative is 1/2, do not occur in random data)
    gated = O.relu_grad(np.where(fused_y > 0, 1.0, -1.0), dy)
    fdx, fdg, fdb = O.batchnorm_backward(gated.astype(np.float32), x, gamma, eps)
    assert_close(dx.asnumpy(), fdx, 1e-4, "bn+relu dx")
    assert_close(dg.asnumpy().ravel(), fdg, 1e-4, "bn+relu dgamma")
    assert_close(db.asnumpy().ravel(), fdb, 1e-4, "bn+relu dbeta")


def _ce_cases(seed, count):
    rng = np.random.RandomState(seed)
    return [(int(rng.choice([1, 2, 7, 64, 300])), int(rng.choice([1, 2, 10, 33, 1000, 1001, 2048, 2050, 2052, 4096, 32000])))
            for _ in range(count)]


@pytest.mark.parametrize("rows,cols", sorted(set(_ce_cases(9, 60))))
def test_random_softmax_cross_entropy(rows, cols):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState(rows * 1009 + cols)
    logits = (rng.normal(size=(rows, cols)) * 3).astype(np.float32)
    labels = np.zeros((rows, cols), np.float32)
    labels[np.arange(rows), rng.randint(0, cols, rows)] = 1.0
    if cols > 1 and rows % 2 == 0:                        # smoothed labels on half of the cases
        labels = (labels * 0.9 + 0.1 / cols).astype(np.float32)
    g = np.array([rng.uniform(0.5, 2.0)], np.float32)
    arr = lambda a: ndarray.array(a, ctx)
    gl, gy, gg = arr(logits), arr(labels), arr(g)
    loss, grad, sm = ndarray.empty((1,), ctx), ndarray.empty((rows, cols), ctx), ndarray.empty((rows, cols), ctx)
    L.softmax_cross_entropy(gl, gy, loss)
    L.softmax_cross_entropy_gradient(gl, gy, gg, grad)
    L.softmax(gl, sm)
    # the loss is a difference of terms the size of the logits (log-sum-exp minus the label's logit): a
    # confident row gives a loss far below them, so the error is measured against their scale as well
    ref_loss = float(np.asarray(O.softmax_ce(logits, labels)).reshape(-1)[0])
    assert abs(float(loss.asnumpy()[0]) - ref_loss) <= 1e-4 * max(abs(ref_loss), 1e-2 * float(np.abs(logits).max()))
    assert_close(grad.asnumpy(), O.softmax_ce_grad(logits, labels, g), 1e-4, "ce grad")
    assert_close(sm.asnumpy(), O.softmax(logits), 1e-4, "softmax")


def _shape(rng, ndim, big):
    ext = [1, 2, 3, 4, 5, 7, 8, 16, 17, 33, 64, 65] + ([130, 257] if big else [])
    while True:
        s = tuple(int(rng.choice(ext)) for _ in range(ndim))
        if np.prod(s) <= 2_000_000:
            return s


def _layout_cases(seed, count):
    rng = np.random.RandomState(seed)
    return [(_shape(rng, int(rng.randint(1, 6)), rng.rand() < 0.3), int(rng.randint(1 << 30))) for _ in range(count)]


@pytest.mark.parametrize("shape,seed", _layout_cases(21, 120))
def test_random_layout_ops(shape, seed):
    """Transpose with a random permutation, reduce-sum over a random axis subset, concat and slice along
    a random axis with their gradients, constant padding: data movement is bit-exact, sums 1e-4."""
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState(seed)
    nd = len(shape)
    x = rng.normal(size=shape).astype(np.float32)
    gx = ndarray.array(x, ctx)
    # transpose
    perm = tuple(int(p) for p in rng.permutation(nd))
    ref = O.transpose(x, perm)
    out = ndarray.empty(ref.shape, ctx)
    L.matrix_transpose(gx, out, perm)
    np.testing.assert_array_equal(out.asnumpy(), ref)
    # reduce-sum
    axes = sorted(int(a) for a in rng.choice(nd, size=rng.randint(1, nd + 1), replace=False))
    ref = O.reduce_sum(x, axes)
    out = ndarray.empty(ref.shape or (1,), ctx)
    L.reduce_sum(gx, out, axes)
    assert_close(out.asnumpy().reshape(ref.shape), ref, 1e-4, f"reduce_sum {shape} {axes}")
    # concat with a second array that differs along the axis, and the gradients back
    axis = int(rng.randint(nd))
    sb = list(shape)
    sb[axis] = int(rng.choice([1, 2, 5, 16, 33]))
    b = rng.normal(size=sb).astype(np.float32)
    ref = O.concat(x, b, axis)
    out = ndarray.empty(ref.shape, ctx)
    L.concat(gx, ndarray.array(b, ctx), out, axis)
    np.testing.assert_array_equal(out.asnumpy(), ref)
    ga, gb = ndarray.empty(shape, ctx), ndarray.empty(tuple(sb), ctx)
    L.concat_gradient(out, ga, axis, 0)
    L.concat_gradient(out, gb, axis, 1)
    np.testing.assert_array_equal(ga.asnumpy(), x)
    np.testing.assert_array_equal(gb.asnumpy(), b)
    # slice a random box out of the concatenated array, and scatter it back into zeros
    begin = [int(rng.randint(0, e)) for e in ref.shape]
    size = [int(rng.randint(1, e - b0 + 1)) for e, b0 in zip(ref.shape, begin)]
    box = ndarray.empty(tuple(size), ctx)
    L.matrix_slice(out, box, begin)
    np.testing.assert_array_equal(box.asnumpy(), O.slice_(ref, begin, size))
    back = ndarray.empty(ref.shape, ctx)
    L.matrix_slice_gradient(box, back, begin)
    np.testing.assert_array_equal(back.asnumpy(), O.slice_grad(box.asnumpy(), begin, ref.shape))
    # constant padding of the trailing axes of a 4-D array
    if nd == 4:
        k = int(rng.randint(0, 5))
        paddings = [(int(rng.randint(0, 4)), int(rng.randint(0, 4))) for _ in range(k)]
        ref = O.pad(x, paddings, 0.25)
        out = ndarray.empty(ref.shape, ctx)
        L.pad(gx, out, paddings, "CONSTANT", 0.25)
        np.testing.assert_array_equal(out.asnumpy(), ref.astype(np.float32))
        dx = ndarray.empty(shape, ctx)
        L.pad_gradient(out, dx, paddings, "CONSTANT")
        np.testing.assert_array_equal(dx.asnumpy(), x)
