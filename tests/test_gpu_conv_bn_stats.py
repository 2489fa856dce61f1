"""Convolution that hands its output's batch statistics to the BatchNorm behind it
(TSplit_Conv2dBatchNormStats / TSplit_BatchNormFromStats), through the C ABI.

Bars: the convolution's output is bit-identical to CuDNN_DLGpuConv2d's; the sums equal the float64 sums
of that output to 1e-5 of their magnitude; BatchNorm(+Relu) from the sums meets the oracle's BatchNorm
of the same activations within 1e-4 (max error over max magnitude), the tolerance stated for BatchNorm."""
import numpy as np
import pytest

from oracle import nets, ops as O
from util import assert_close

pytestmark = pytest.mark.gpu

# (N, C, H, W, O, k, pad, stride, forced routing or None): every forward route of the library
CASES = [
    (4, 3, 20, 20, 24, 3, 1, 1, None),        # thin first layer (vector ALU kernel): sums by a pass over y
    (3, 24, 9, 9, 20, 3, 1, 1, None),         # generic gather engine (C not a multiple of 16)
    (4, 64, 32, 32, 64, 3, 1, 1, "0"),        # tap-major, 64 x 256 tiles, cut tiles assembled by the second kernel
    (2, 32, 17, 17, 40, 3, 1, 1, "0"),        # tap-major, 64-row tiles, ragged columns (289 positions per image)
    (5, 48, 14, 14, 136, 3, 1, 1, "0"),       # tap-major, 128 x 128 tiles, two row tiles, ragged rows
    (3, 16, 40, 40, 192, 1, 0, 1, None),      # 1x1 filter used where it lies
    (2, 32, 23, 19, 72, 3, 1, 2, None),       # stride 2
    (64, 64, 56, 56, 64, 3, 1, 1, "0"),       # tap-major with thousands of tiles (the three-block variant)
    (4, 128, 28, 28, 128, 3, 1, 1, "1"),      # Winograd, whole 4x4 tiles
    (3, 64, 30, 26, 80, 3, 1, 1, "1"),        # Winograd, planes that the 4x4 tiling overhangs
    (16, 128, 56, 56, 256, 3, 1, 1, None),    # Winograd by the library's own choice
]


def _ctx():
    from tsplit_amd import gpu_links as L, ndarray
    return L, ndarray, ndarray.gpu(0)


def _stats_rows(stats, slots, C):
    return stats.asnumpy().view(np.float64).reshape(-1, C, 2)[:slots]


@pytest.mark.parametrize("case", CASES)
def test_conv_output_is_unchanged_and_sums_are_the_outputs(case, rng, monkeypatch):
    L, nd, ctx = _ctx()
    N, C, H, W, Oc, k, pad, s, forced = case
    if forced is not None:
        monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", forced)
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, k, k)) / np.sqrt(C * k * k)).astype(np.float32)
    oh, ow = (H + 2 * pad - k) // s + 1, (W + 2 * pad - k) // s + 1
    gx, gw = nd.array(x, ctx), nd.array(w, ctx)
    y0, y1 = nd.empty((N, Oc, oh, ow), ctx), nd.empty((N, Oc, oh, ow), ctx)
    # three rows, the middle one written: its neighbours must stay as they were
    stats = nd.array(np.full((3 * Oc * 4,), 7.0, np.float32), ctx)
    L.CuDNN_conv2d(gx, gw, y0, pad, pad, s)
    L.conv2d_batch_norm_stats(gx, gw, y1, stats, 1, pad, pad, s)
    plain, got = y0.asnumpy(), y1.asnumpy()
    np.testing.assert_array_equal(got, plain)
    if N * C * H * W <= 1 << 22:          # the oracle's convolution on the cases it finishes in seconds
        assert_close(got, O.conv2d(x, w, pad, pad, s), 2e-3, f"conv {case}")
    rows = stats.asnumpy().view(np.float64).reshape(3, Oc, 2)
    seven = np.full((Oc * 4,), 7.0, np.float32).view(np.float64).reshape(Oc, 2)
    np.testing.assert_array_equal(rows[0], seven)
    np.testing.assert_array_equal(rows[2], seven)
    y64 = got.astype(np.float64)
    want_sum, want_sq = y64.sum(axis=(0, 2, 3)), (y64 * y64).sum(axis=(0, 2, 3))
    scale = np.abs(y64).sum(axis=(0, 2, 3)).max()
    assert np.abs(rows[1][:, 0] - want_sum).max() <= 1e-5 * scale, np.abs(rows[1][:, 0] - want_sum).max() / scale
    assert np.abs(rows[1][:, 1] - want_sq).max() <= 1e-5 * want_sq.max()


@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("case,pieces", [((8, 32, 16, 16, 48, 3, 1, 1, "0"), 4), ((8, 64, 12, 12, 64, 3, 1, 1, "1"), 2),
                                         ((6, 3, 10, 10, 16, 3, 1, 1, None), 3), ((4, 16, 9, 9, 24, 3, 1, 1, None), 1)])
def test_batchnorm_from_the_sums_of_micro_tensor_convolutions(case, pieces, relu, rng, monkeypatch):
    """The convolution runs on `pieces` batch micro-tensors, each writing its own row of sums; the
    BatchNorm behind it sees the whole batch and must equal the oracle's BatchNorm of the whole output."""
    L, nd, ctx = _ctx()
    N, C, H, W, Oc, k, pad, s, forced = case
    if forced is not None:
        monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", forced)
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, k, k)) / np.sqrt(C * k * k) * 3).astype(np.float32)
    gamma = rng.normal(size=(1, Oc, 1, 1)).astype(np.float32)
    beta = rng.normal(size=(1, Oc, 1, 1)).astype(np.float32)
    eps = 0.01
    gx, gw = nd.array(x, ctx), nd.array(w, ctx)
    y, z = nd.empty((N, Oc, H, W), ctx), nd.empty((N, Oc, H, W), ctx)
    gx.split_tensor(pieces)
    y.split_tensor(pieces)
    stats = nd.empty((pieces * Oc * 4,), ctx)
    for i in range(pieces):
        L.conv2d_batch_norm_stats(gx.sTensor[i], gw, y.sTensor[i], stats, i, pad, pad, s)
    sm, sv = nd.empty((1, Oc, 1, 1), ctx), nd.empty((1, Oc, 1, 1), ctx)
    L.batch_norm_from_stats(y, stats, pieces, nd.array(gamma, ctx), nd.array(beta, ctx), z, sm, sv, eps, relu)
    conv_out = y.asnumpy()
    assert_close(conv_out, O.conv2d(x, w, pad, pad, s), 2e-3, "conv on micro-tensors")
    ref, mean, var = O.batchnorm_forward(conv_out, gamma, beta, eps)
    if relu:
        ref = O.relu(ref)
    assert_close(z.asnumpy(), ref, 1e-4, "BatchNorm from the convolution's sums")
    assert_close(sm.asnumpy().ravel(), mean, 1e-4, "saved mean")
    assert_close(sv.asnumpy().ravel(), 1 / np.sqrt(var + eps), 1e-4, "saved inverse deviation")
    # and it agrees with the library's own two-pass BatchNorm of the same activations
    z2 = nd.empty((N, Oc, H, W), ctx)
    if relu:
        L.batch_norm_relu(y, nd.array(gamma, ctx), nd.array(beta, ctx), z2, sm, sv, eps)
    else:
        L.CuDNN_Batch_Normalization(y, nd.array(gamma, ctx), nd.array(beta, ctx), z2, sm, sv, 0.99, eps)
    assert_close(z.asnumpy(), z2.asnumpy(), 2e-5, "one-pass against two-pass BatchNorm")


def test_statistics_argument_errors():
    L, nd, ctx = _ctx()
    x, w = nd.array(np.zeros((2, 16, 8, 8), np.float32), ctx), nd.array(np.zeros((8, 16, 3, 3), np.float32), ctx)
    y = nd.empty((2, 8, 8, 8), ctx)
    small = nd.empty((8 * 4 - 1,), ctx)
    with pytest.raises(Exception):
        L.conv2d_batch_norm_stats(x, w, y, small, 0, 1, 1, 1)
    ok = nd.empty((8 * 4,), ctx)
    with pytest.raises(Exception):
        L.conv2d_batch_norm_stats(x, w, y, ok, 1, 1, 1, 1)          # row 1 does not exist
    g = nd.array(np.ones((1, 8, 1, 1), np.float32), ctx)
    with pytest.raises(Exception):
        L.batch_norm_from_stats(y, ok, 2, g, g, y, None, None, 0.01, False)     # two rows asked, one held
    with pytest.raises(Exception):
        L.batch_norm_from_stats(y, ok, 1, g, g, y, None, None, 0.01, True)      # the fused form needs the save arrays


def _onehot(lab, n):
    out = np.zeros((len(lab), n), np.float32)
    out[np.arange(len(lab)), lab] = 1
    return out


@pytest.mark.parametrize("split,fuse", [(None, False), ({0: 4, 3: 2}, False), ({0: 4, 3: 4}, True)])
def test_training_with_statistics_from_the_convolutions_tracks_oracle(split, fuse):
    """The small conv net of the end-to-end tests, six momentum steps against the oracle, with every
    BatchNorm taking its statistics from the convolution in front of it."""
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
    t = trainer.Trainer(spec, params, X.shape, 10, ctx, optimizer=("momentum", 0.05, 0.9), split=split,
                        fuse_bn_relu=fuse, conv_bn_stats=True)
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for _ in range(6):
        t.step(gx, gy)
        losses.append(t.loss_value())
    rel = np.max(np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses))
    assert rel <= 1e-3, (rel, losses, ref_losses)
    for k in params:
        assert_close(t.params[k].asnumpy(), ref_params[k], 2e-3, k)
