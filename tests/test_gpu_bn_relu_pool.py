"""BatchNorm + Relu + 2x2 / stride 2 max pooling as one call each way (TSplit_BatchNormReluMaxPool,
TSplit_BatchNormReluMaxPoolFromStats, TSplit_BatchNormReluMaxPool_gradient), through the C ABI.

Bars: the pooled output equals, bit for bit, what TSplit_BatchNormRelu followed by CuDNN_DLGpuMax_Pooling2d gives
where that runs its two-pass kernels (same float expressions, and a maximum does not depend on the order it is
taken in; within 2e-6 for the small channels that take its one-pass kernel) and meets the oracle's
BatchNorm -> Relu -> max pooling within 1e-4 (max error over max magnitude, the tolerance stated for BatchNorm);
the gradients meet the oracle's chain max_pool_grad -> relu_grad -> batchnorm_backward within 1e-4 and the
library's own three-call chain within 2e-5, including windows whose values tie (all non-positive under the
Relu: the gradient goes to the first element and is gated there)."""
import numpy as np
import pytest

from oracle import nets, ops as O
from util import assert_close

pytestmark = pytest.mark.gpu

# N, C, H, W
SHAPES = [
    (4, 16, 8, 8),        # 16-byte words, channels small enough for one block each
    (3, 5, 6, 10),        # rows of 10: 8-byte words
    (2, 3, 14, 14),       # rows of 14 (the last VGG stage): 8-byte words
    (2, 64, 28, 28),
    (8, 32, 56, 56),      # several ranges per channel in the gradient's sums
    (16, 64, 112, 112),   # a VGG stage end at a quarter of its batch
]


def _ctx():
    from tsplit_amd import gpu_links as L, ndarray
    return L, ndarray, ndarray.gpu(0)


def _inputs(shape, rng):
    N, C, H, W = shape
    x = rng.normal(size=shape).astype(np.float32)
    # whole windows below zero in places, so that ties under the Relu occur in every channel
    x[:, :, : H // 2 : 2, ::3] -= 4.0
    gamma = rng.uniform(0.5, 1.5, size=(1, C, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, C, 1, 1)).astype(np.float32) * 0.3
    dyp = rng.normal(size=(N, C, H // 2, W // 2)).astype(np.float32)
    return x, gamma, beta, dyp


@pytest.mark.parametrize("shape", SHAPES)
def test_forward_and_gradient_against_oracle_and_three_calls(shape, rng):
    L, nd, ctx = _ctx()
    N, C, H, W = shape
    eps = 0.01
    x, gamma, beta, dyp = _inputs(shape, rng)
    gx, gg, gb, gdyp = nd.array(x, ctx), nd.array(gamma, ctx), nd.array(beta, ctx), nd.array(dyp, ctx)
    # the three calls
    a = nd.empty(shape, ctx)
    sm0, sv0 = nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.batch_norm_relu(gx, gg, gb, a, sm0, sv0, eps)
    p0 = nd.empty(dyp.shape, ctx)
    L.CuDNN_max_pooling2d(a, 2, 2, p0, 0, 2)
    da = nd.empty(shape, ctx)
    L.CuDNN_max_pooling2d_gradient(p0, gdyp, a, 2, 2, da, 0, 2)
    dx0, dg0, db0 = nd.empty(shape, ctx), nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.batch_norm_relu_gradient(da, gx, gg, gb, dx0, dg0, db0, sm0, sv0, eps)
    # the one call
    p1 = nd.empty(dyp.shape, ctx)
    sm1, sv1 = nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.batch_norm_relu_max_pool(gx, gg, gb, p1, sm1, sv1, eps)
    if N * H * W > 64 * 256:
        np.testing.assert_array_equal(p1.asnumpy(), p0.asnumpy())
        np.testing.assert_array_equal(sm1.asnumpy(), sm0.asnumpy())
        np.testing.assert_array_equal(sv1.asnumpy(), sv0.asnumpy())
    else:   # channels of at most 16 384 values take a one-pass kernel in the two-call form: other roundings
        assert_close(p1.asnumpy(), p0.asnumpy(), 2e-6, "pooled output against the three calls")
        assert_close(sm1.asnumpy(), sm0.asnumpy(), 2e-6, "saved mean against the three calls")
        assert_close(sv1.asnumpy(), sv0.asnumpy(), 2e-6, "saved inverse deviation against the three calls")
    dx1, dg1, db1 = nd.empty(shape, ctx), nd.empty((1, C, 1, 1), ctx), nd.empty((1, C, 1, 1), ctx)
    L.batch_norm_relu_max_pool_gradient(gdyp, gx, gg, gb, dx1, dg1, db1, sm1, sv1, eps)
    assert_close(dx1.asnumpy(), dx0.asnumpy(), 2e-5, "dx against the three calls")
    assert_close(dg1.asnumpy(), dg0.asnumpy(), 2e-5, "dscale against the three calls")
    assert_close(db1.asnumpy(), db0.asnumpy(), 2e-5, "dbias against the three calls")
    # the oracle's chain
    if N * C * H * W <= 1 << 21:
        y, mean, var = O.batchnorm_forward(x, gamma, beta, eps)
        act = O.relu(y)
        pooled = O.max_pool(act, 2, 2, 0, 2)
        assert_close(p1.asnumpy(), pooled, 1e-4, "pooled output")
        d_act = O.max_pool_grad(act, dyp, 2, 2, 0, 2)
        d_y = O.relu_grad(y, d_act)
        dx, dgam, dbet = O.batchnorm_backward(d_y, x, gamma, eps)
        assert_close(dx1.asnumpy(), dx, 1e-4, "dx")
        assert_close(dg1.asnumpy().ravel(), np.asarray(dgam).ravel(), 1e-4, "dscale")
        assert_close(db1.asnumpy().ravel(), np.asarray(dbet).ravel(), 1e-4, "dbias")


def test_statistics_from_a_convolution(rng, monkeypatch):
    """The convolution leaves the sums (two micro-tensors, two rows), the fused call takes them."""
    L, nd, ctx = _ctx()
    N, C, H, W, Oc = 8, 16, 12, 12, 24
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, 3, 3)) / np.sqrt(C * 9) * 3).astype(np.float32)
    gamma = rng.normal(size=(1, Oc, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, Oc, 1, 1)).astype(np.float32)
    gx, gw = nd.array(x, ctx), nd.array(w, ctx)
    y = nd.empty((N, Oc, H, W), ctx)
    gx.split_tensor(2)
    y.split_tensor(2)
    stats = nd.empty((2 * Oc * 4,), ctx)
    for i in range(2):
        L.conv2d_batch_norm_stats(gx.sTensor[i], gw, y.sTensor[i], stats, i, 1, 1, 1)
    pooled = nd.empty((N, Oc, H // 2, W // 2), ctx)
    sm, sv = nd.empty((1, Oc, 1, 1), ctx), nd.empty((1, Oc, 1, 1), ctx)
    L.batch_norm_relu_max_pool(y, nd.array(gamma, ctx), nd.array(beta, ctx), pooled, sm, sv, 0.01, stats=stats, slots=2)
    conv_out = y.asnumpy()
    ref, mean, var = O.batchnorm_forward(conv_out, gamma, beta, 0.01)
    assert_close(pooled.asnumpy(), O.max_pool(O.relu(ref), 2, 2, 0, 2), 1e-4, "pooled output from the convolution's sums")
    assert_close(sm.asnumpy().ravel(), mean, 1e-4, "saved mean")


def test_argument_errors():
    L, nd, ctx = _ctx()
    x = nd.array(np.zeros((2, 4, 6, 7), np.float32), ctx)          # odd width
    g = nd.array(np.ones((1, 4, 1, 1), np.float32), ctx)
    s1, s2 = nd.empty((1, 4, 1, 1), ctx), nd.empty((1, 4, 1, 1), ctx)
    with pytest.raises(Exception):
        L.batch_norm_relu_max_pool(x, g, g, nd.empty((2, 4, 3, 3), ctx), s1, s2)
    x = nd.array(np.zeros((2, 4, 6, 8), np.float32), ctx)
    with pytest.raises(Exception):
        L.batch_norm_relu_max_pool(x, g, g, nd.empty((2, 4, 3, 3), ctx), s1, s2)        # wrong pooled shape
    with pytest.raises(Exception):
        L.batch_norm_relu_max_pool_gradient(nd.empty((2, 4, 3, 3), ctx), x, g, g, nd.empty((2, 4, 6, 8), ctx), s1, s2, s1, s2)
    # statistics over an empty batch are refused, as the BatchNorm entry points refuse them
    e, pe = nd.empty((0, 4, 6, 8), ctx), nd.empty((0, 4, 3, 4), ctx)
    with pytest.raises(Exception):
        L.batch_norm_relu_max_pool(e, g, g, pe, s1, s2)
    with pytest.raises(Exception):
        L.batch_norm_relu_max_pool_gradient(pe, e, g, g, nd.empty((0, 4, 6, 8), ctx), s1, s2, s1, s2)
    # and the library still works
    p = nd.empty((2, 4, 3, 4), ctx)
    L.batch_norm_relu_max_pool(x, g, g, p, s1, s2)
    np.testing.assert_allclose(p.asnumpy(), 1.0)      # zeros normalise to zero, plus a bias of one


def _onehot(lab, n):
    out = np.zeros((len(lab), n), np.float32)
    out[np.arange(len(lab)), lab] = 1
    return out


@pytest.mark.parametrize("stats", [False, True])
def test_training_with_the_fused_stage_ends_tracks_oracle(stats):
    """The small conv net of the end-to-end tests, six momentum steps against the oracle, with both stage ends
    (BatchNorm, Relu, max pooling) as one call each way."""
    from tsplit_amd import ndarray, trainer
    rng = np.random.RandomState(7)
    spec = [("conv", "c1", 3, 8, 3, 1, 1), ("bn", "c1_bn", 8), ("relu",),
            ("conv", "c2", 8, 16, 3, 1, 1), ("bn", "c2_bn", 16), ("relu",), ("maxpool", 2, 0, 2),
            ("conv", "c3", 16, 16, 3, 1, 1), ("bn", "c3_bn", 16), ("relu",), ("maxpool", 2, 0, 2),
            ("flatten",), ("fc", "f1", 16 * 4 * 4, 32), ("fc", "f2", 32, 10)]
    X = rng.normal(size=(8, 3, 16, 16)).astype(np.float32)
    Y = _onehot(rng.randint(0, 10, 8), 10)
    params = trainer.init_params(spec, seed=5)
    ref_losses, ref_params = nets.train(spec, params, X, Y, steps=6, lr=0.05, momentum=0.9)
    ctx = ndarray.gpu(0)
    t = trainer.Trainer(spec, params, X.shape, 10, ctx, optimizer=("momentum", 0.05, 0.9), split={0: 4, 3: 2},
                        fuse_bn_relu=True, conv_bn_stats=stats, fuse_max_pool=True)
    assert len(t.fused_pool) == 2
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for _ in range(6):
        t.step(gx, gy)
        losses.append(t.loss_value())
    rel = np.max(np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses))
    assert rel <= 1e-3, (rel, losses, ref_losses)
    for k in params:
        assert_close(t.params[k].asnumpy(), ref_params[k], 2e-3, k)
