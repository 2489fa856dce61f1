"""Every distinct convolution of full-size VGG-16 (batch 64, 224x224, the first four layers on the
16-image micro-tensors the benchmark step gives them), ResNet-50 (batch 64, 224x224) and Inception-v4
(batch 32, 299x299), as `tsplit_amd.workloads` builds them from the reference's examples
(examples/imagenet_vgg.py:24-98, examples/imagenet_resnet.py:26-122,
examples/imagenet_inceptionv4.py:84-234), through all three passes at the FULL batch, so that the
kernels, tile shapes and cuts between blocks under test are the ones a training step of those nets
launches:

  * forward and data gradient of the first two images and the last one against the float64 oracle
    (images are independent, so a few images of the full-batch result pin the launch),
  * the filter gradient, which sums over the batch: a block of 8 x 8 channel pairs of the full-batch
    result against the oracle run on those channels of the whole batch, the adjoint identity
    <conv(x, w), dy> = <x, dx> = <w, dw> evaluated in float64 on the host, and the whole gradient
    against the oracle on a two-image batch of the same geometry,
  * for VGG-16 every layer but the three-channel first one must take the Winograd routine in all
    three passes (as in the benchmark step), so none of this can pass on another kernel,

then one full-size training step of each branched example network (ResNet-50, Inception-v4, the
Transformer): finite loss, a gradient for every parameter, and the same bits when the step is repeated.
Tolerances: 2e-3 of the largest entry for convolutions (measured ~1e-6); inner products to 1e-4 of
the product of the norms.
"""
import numpy as np
import pytest

from oracle import ops as O
from tsplit_amd import workloads
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 2e-3

GEOMETRIES = [("vgg16",) + g for g in workloads.conv_geometries("vgg16")] + \
             [("resnet50",) + g for g in workloads.conv_geometries("resnet50")] + \
             [("inception_v4",) + g for g in workloads.conv_geometries("inception_v4")]


def _dot64(a, b):
    return float(np.sum(a.astype(np.float64).ravel() * b.ravel()))


def _norm64(a):
    return float(np.sqrt(np.sum(np.square(a.astype(np.float64)))))


def _three_passes(x, w, dy, ph, pw, s):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    y, dx, dw = ndarray.empty(dy.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
    L.CuDNN_conv2d(gx, gw, y, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, ph, pw, s)
    return y.asnumpy(), dx.asnumpy(), dw.asnumpy()


@pytest.mark.parametrize("geo", GEOMETRIES, ids=lambda g: "%s-n%d-c%d-%dx%d-o%d-k%dx%d-p%d%d-s%d" % g)
def test_full_size_convolution(geo):
    net, N, C, H, W, Oc, kH, kW, ph, pw, s = geo
    rng = np.random.default_rng(abs(hash(geo[1:])) % (1 << 31))
    oH, oW = (H + 2 * ph - kH) // s + 1, (W + 2 * pw - kW) // s + 1
    x = rng.standard_normal((N, C, H, W), dtype=np.float32)
    w = (rng.standard_normal((Oc, C, kH, kW), dtype=np.float32) / np.float32(np.sqrt(C * kH * kW)))
    dy = rng.standard_normal((N, Oc, oH, oW), dtype=np.float32)
    if net == "vgg16" and C >= 64:
        from tsplit_amd import gpu_links as L
        assert L.conv_takes_winograd(N, C, Oc, H, W), geo
        assert L.conv_takes_winograd(N, C, Oc, H, W, data_gradient=True), geo
        assert L.conv_takes_winograd(N, C, Oc, H, W, filter_gradient=True), geo
    y, dx, dw = _three_passes(x, w, dy, ph, pw, s)
    # a few images of the full-batch launches against the oracle
    pick = [0, 1, N - 1]
    assert_close(y[pick], O.conv2d(x[pick], w, ph, pw, s), TOL, "forward %s" % (geo,))
    assert_close(dx[pick], O.conv2d_grad_data(w, dy[pick], x[pick].shape, ph, pw, s), TOL, "data gradient %s" % (geo,))
    # a block of the full-batch filter gradient: the sum over all images for 8 x 8 channel pairs
    cs, os_ = np.sort(rng.choice(C, min(C, 8), replace=False)), np.sort(rng.choice(Oc, min(Oc, 8), replace=False))
    block = O.conv2d_grad_filter(np.ascontiguousarray(x[:, cs]), np.ascontiguousarray(dy[:, os_]),
                                 (len(os_), len(cs), kH, kW), ph, pw, s)
    assert_close(dw[np.ix_(os_, cs)], block, TOL, "filter gradient over the whole batch, channel block %s" % (geo,))
    # the three passes are one bilinear form: <y, dy> = <x, dx> = <w, dw>
    form = _dot64(y, dy)
    scale = _norm64(y) * _norm64(dy)
    assert abs(_dot64(x, dx) - form) <= 1e-4 * scale, (geo, form, _dot64(x, dx))
    assert abs(_dot64(w, dw) - form) <= 1e-4 * scale, (geo, form, _dot64(w, dw))
    # the filter gradient against the oracle: a two-image batch of the same geometry
    _, _, dw2 = _three_passes(x[:2], w, dy[:2], ph, pw, s)
    assert_close(dw2, O.conv2d_grad_filter(x[:2], dy[:2], w.shape, ph, pw, s), TOL, "filter gradient %s" % (geo,))


def _step_twice(build, inputs, seed):
    """Two runs of forward + backward from the same parameters -> ((loss, grads), (loss, grads), store)."""
    from tsplit_amd import graph, ndarray, stream
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    backend = graph.GpuBackend(ctx, st)
    store = workloads.ParamStore(seed)
    runs = []
    for _ in range(2):
        t = graph.Tape(backend)
        b = workloads.Binder(t, store)
        dev = {k: b.input(v) for k, v in inputs.items()}
        loss, _ = build(t, b, dev)
        t.backward(loss)
        backend.sync()
        runs.append((float(loss.value.asnumpy()[0]), b.grads()))
    return runs[0], runs[1], store


def _check_step(first, second, store, order_dependent=()):
    (l1, g1), (l2, g2) = first, second
    assert np.isfinite(l1) and l1 > 0
    assert set(g1) == {k for k, tr in store.trainable.items() if tr}       # every parameter received a gradient
    for k, g in g1.items():
        assert np.isfinite(g).all(), k
        assert np.any(g != 0), "gradient of %s is all zero" % k
    assert l1 == l2
    for k in g1:
        if k in order_dependent:
            assert_close(g2[k], g1[k], 1e-5, k)
        else:
            assert np.array_equal(g1[k], g2[k]), k


def _images(rng, n, hw, classes=1000):
    x = rng.standard_normal((n, 3, hw, hw), dtype=np.float32)
    y = np.zeros((n, classes), np.float32)
    y[np.arange(n), rng.integers(0, classes, n)] = 1
    return {"x": x, "y": y}


def test_resnet50_full_size_step():
    """ResNet-50, batch 64, 224x224, 1000 classes (examples/imagenet_resnet.py:88-122)."""
    first, second, store = _step_twice(lambda t, b, d: workloads.resnet(t, b, d["x"], d["y"]),
                                       _images(np.random.default_rng(1), 64, 224), seed=123)
    _check_step(first, second, store)
    assert abs(first[0] - np.log(1000.0)) < 6.0          # He init, random labels: log(classes) and a few units


def test_inception_v4_full_size_step():
    """Inception-v4, batch 32, 299x299, 1000 classes (examples/imagenet_inceptionv4.py:189-253)."""
    first, second, store = _step_twice(lambda t, b, d: workloads.inception_v4(t, b, d["x"], d["y"]),
                                       _images(np.random.default_rng(2), 32, 299), seed=123)
    _check_step(first, second, store)
    assert abs(first[0] - np.log(1000.0)) < 6.0


def test_transformer_full_size_step():
    """Encoder-decoder, 6+6 blocks, d_model 512, 8 heads, FFN 2048, length 256, batch 32, vocabulary
    32 000 (examples/transformer.py:215-287).  The graph has no softmax or layer norm in its attention,
    so masked scores are filled with 0 and the embeddings are small, which keeps twelve blocks finite;
    shapes and operator sequence are the example's.  The embedding table's gradient is a scatter-add
    with float atomics: repeatable to rounding, not to the bit."""
    rng = np.random.default_rng(3)
    cfg = workloads.TransformerConfig(batch=32, mask_value=0.0, embed_std=0.0002, pos_amplitude=0.003)
    inputs = {"xs": rng.integers(1, cfg.vocab, size=(32, cfg.len1)).astype(np.float32),
              "yi": rng.integers(1, cfg.vocab, size=(32, cfg.len2)).astype(np.float32),
              "yo": rng.integers(1, cfg.vocab, size=(32, cfg.len2)).astype(np.float32)}
    first, second, store = _step_twice(lambda t, b, d: workloads.transformer(t, b, cfg, d["xs"], d["yi"], d["yo"]),
                                       inputs, seed=123)
    _check_step(first, second, store, order_dependent=("embedding_table",))
    assert abs(first[0] - np.log(32000.0)) < 6.0
