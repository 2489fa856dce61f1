"""The streaming operators at the full size of the benchmark's largest activation
(64 x 64 x 224 x 224, 822 MB) and of its largest parameter (25088 x 4096): values that numpy gives
exactly (Relu, its gradient, 2x2 max pooling) are compared bit for bit; BatchNorm is checked through
its invariants and float64 per-channel statistics; the momentum update against the fp32 recurrence."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SHAPE = (64, 64, 224, 224)


@pytest.fixture(scope="module")
def big():
    from tsplit_amd import ndarray
    rng = np.random.RandomState(42)
    base = rng.standard_normal((8,) + SHAPE[1:]).astype(np.float32)        # 103 MB of normals, tiled 8 times
    x = np.concatenate([base * (1.0 + 0.125 * i) + 0.01 * i for i in range(8)], axis=0)
    ctx = ndarray.gpu(0)
    return {"x": x, "gx": ndarray.array(x, ctx), "ctx": ctx, "nd": ndarray}


def test_relu_and_gradient_bit_exact(big):
    from tsplit_amd import gpu_links as L
    nd, ctx, x = big["nd"], big["ctx"], big["x"]
    y = nd.empty(SHAPE, ctx)
    L.relu(big["gx"], y)
    assert np.array_equal(y.asnumpy(), np.maximum(x, 0))
    dy = np.roll(x, 12345).reshape(SHAPE)                                   # any other values
    gdy = nd.array(dy, ctx)
    L.relu_gradient(big["gx"], gdy, y)
    assert np.array_equal(y.asnumpy(), np.where(x > 0, dy, np.where(x == 0, np.float32(0.5) * dy, np.float32(0))))


def test_max_pool_2x2_bit_exact_and_routing(big):
    from tsplit_amd import gpu_links as L
    nd, ctx, x = big["nd"], big["ctx"], big["x"]
    N, C, H, W = SHAPE
    y = nd.empty((N, C, H // 2, W // 2), ctx)
    L.max_pooling2d(big["gx"], 2, 2, y, 0, 2)
    ref = x.reshape(N, C, H // 2, 2, W // 2, 2).max(axis=(3, 5))
    got = y.asnumpy()
    assert np.array_equal(got, ref)
    # backward: every window hands its gradient to exactly one element, the one holding the maximum
    dy = np.abs(ref) + 1.0
    dx = nd.empty(SHAPE, ctx)
    L.max_pooling2d_gradient(big["gx"], nd.array(dy, ctx), 2, 2, dx, 0, 2)
    gdx = dx.asnumpy()
    win = gdx.reshape(N, C, H // 2, 2, W // 2, 2)
    assert np.array_equal(win.sum(axis=(3, 5)), dy)
    assert np.array_equal((win != 0).sum(axis=(3, 5)), np.ones_like(dy, dtype=np.int64))
    hit = gdx != 0
    assert np.array_equal(x[hit], ref.repeat(2, axis=2).repeat(2, axis=3)[hit])   # ... and it sits on the maximum


def test_batchnorm_statistics_and_invariants(big):
    from tsplit_amd import gpu_links as L
    nd, ctx, x = big["nd"], big["ctx"], big["x"]
    C = SHAPE[1]
    rng = np.random.RandomState(1)
    gamma = rng.uniform(0.5, 1.5, (1, C, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, C, 1, 1)).astype(np.float32)
    eps = 0.01
    y = nd.empty(SHAPE, ctx)
    sm, sv = nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.CuDNN_Batch_Normalization(big["gx"], nd.array(gamma, ctx), nd.array(beta, ctx), y, sm, sv, 0.99, eps)
    mean = x.mean(axis=(0, 2, 3), dtype=np.float64)
    var = x.var(axis=(0, 2, 3), dtype=np.float64)
    np.testing.assert_allclose(sm.asnumpy().ravel(), mean, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(sv.asnumpy().ravel(), 1 / np.sqrt(var + eps), rtol=1e-5)
    gy = y.asnumpy()
    # per channel: mean(y) = beta, var(y) = gamma^2 var / (var + eps)
    np.testing.assert_allclose(gy.mean(axis=(0, 2, 3), dtype=np.float64), beta.ravel(), atol=1e-4)
    np.testing.assert_allclose(gy.var(axis=(0, 2, 3), dtype=np.float64), gamma.ravel().astype(np.float64) ** 2 * var / (var + eps),
                               rtol=1e-4)
    # ... and one image against the closed form
    a = gamma.ravel().astype(np.float64) / np.sqrt(var + eps)
    ref0 = (x[5].astype(np.float64) - mean[:, None, None]) * a[:, None, None] + beta.ravel()[:, None, None]
    assert np.max(np.abs(gy[5] - ref0)) <= 1e-4 * np.max(np.abs(ref0))
    # gradient: dbeta = sum dy, dgamma = sum dy xhat, and dx sums to zero in every channel
    dy = np.ascontiguousarray(np.roll(x, 777, axis=3)[:, ::-1])            # a tensor unrelated to x channel by channel
    del gy
    dx, dg, db = nd.empty(SHAPE, ctx), nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.CuDNN_Batch_Normalization_gradient(nd.array(dy, ctx), big["gx"], nd.array(gamma, ctx), dx, dg, db, sm, sv, eps)
    np.testing.assert_allclose(db.asnumpy().ravel(), dy.sum(axis=(0, 2, 3), dtype=np.float64), rtol=1e-4)
    xhat_dy = np.zeros(C)
    for n in range(SHAPE[0]):                                                # image by image: no 1.6 GB temporaries
        xh = (x[n].astype(np.float64) - mean[:, None, None]) / np.sqrt(var + eps)[:, None, None]
        xhat_dy += (xh * dy[n]).sum(axis=(1, 2))
    np.testing.assert_allclose(dg.asnumpy().ravel(), xhat_dy, rtol=1e-4)
    gdx = dx.asnumpy()
    total = gdx.sum(axis=(0, 2, 3), dtype=np.float64)
    scale = np.abs(gdx).sum(axis=(0, 2, 3), dtype=np.float64)
    assert np.all(np.abs(total) <= 1e-5 * scale)


def test_momentum_update_at_the_largest_parameter():
    from tsplit_amd import gpu_links as L, ndarray as nd
    ctx = nd.gpu(0)
    rng = np.random.RandomState(3)
    n = 25088 * 4096
    p = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    v = rng.standard_normal(n).astype(np.float32) * np.float32(0.1)
    gp, gg, gv = nd.array(p, ctx), nd.array(g, ctx), nd.array(v, ctx)
    lr, mu = np.float32(0.01), np.float32(0.9)
    for _ in range(2):
        L.momentum_update(gp, gg, gv, float(lr), float(mu), False)
        v = (mu * v - lr * g).astype(np.float32)
        p = (p + v).astype(np.float32)
    # fp32 with or without a fused multiply-add: one rounding apart at most
    assert np.max(np.abs(gv.asnumpy() - v)) <= 2e-7 * np.max(np.abs(v))
    assert np.max(np.abs(gp.asnumpy() - p)) <= 2e-7 * np.max(np.abs(p))
