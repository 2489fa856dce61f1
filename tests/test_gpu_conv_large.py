"""Convolutions on tensors beyond what one kernel launch addresses with 32-bit offsets (2 GiB):
forward and backward-data take the gathered tensor in runs of whole images, the filter gradient
addresses each K split from its own first image.  Checked (a) against the CPU oracle on small
shapes with the reach lowered through TSPLIT_CONV_REACH_BYTES so that the same code paths run,
for both tile families, strided phases and ragged image sizes; (b) at real size, a 2.3 GB input,
through properties that need no CPU convolution: a delta filter copies channels exactly, results
equal those of per-image views, and the filter gradient equals the sum of per-image gradients."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 2e-3

# (case, reach bytes): N, C, H, W, O, kH, kW, ph, pw, stride
SMALL = [
    ((7, 16, 20, 20, 32, 3, 3, 1, 1, 1), 120_000),    # forward in runs of 4+3 images, backward-data 2+2+2+1
    ((7, 16, 20, 20, 32, 3, 3, 1, 1, 1), 200_000),    # filter gradient: one image per K split
    ((7, 16, 20, 20, 80, 3, 3, 1, 1, 1), 400_000),    # 128x128 tiles
    ((9, 80, 12, 12, 16, 3, 3, 1, 1, 1), 200_000),    # backward-data on 128x128 tiles
    ((6, 16, 15, 15, 32, 3, 3, 1, 1, 2), 60_000),     # stride 2: every run launches its own phases
    ((5, 16, 7, 7, 24, 3, 3, 1, 1, 1), 16_000),       # 49 positions per image: padded K, straddling words
    ((11, 32, 10, 14, 24, 1, 7, 0, 3, 1), 60_000),    # 1x7, 140 positions
    ((3, 16, 20, 20, 32, 3, 3, 1, 1, 1), 30_000),     # one image per run
    ((3, 16, 20, 20, 32, 3, 3, 1, 1, 1), 20_000),     # not even one image fits: the gather engine takes over
]


@pytest.mark.parametrize("case,reach", SMALL)
def test_runs_of_images_against_the_oracle(case, reach, rng, monkeypatch):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    N, C, H, W, Oc, kH, kW, ph, pw, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, kH, kW)) / np.sqrt(C * kH * kW)).astype(np.float32)
    ref_y = O.conv2d(x, w, ph, pw, s)
    dy = rng.normal(size=ref_y.shape).astype(np.float32)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    y, dx, dw = ndarray.empty(ref_y.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
    monkeypatch.setenv("TSPLIT_CONV_REACH_BYTES", str(reach))
    L.CuDNN_conv2d(gx, gw, y, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, ph, pw, s)
    e1 = assert_close(y.asnumpy(), ref_y, TOL, f"conv fwd {case}")
    e2 = assert_close(dx.asnumpy(), O.conv2d_grad_data(w, dy, x.shape, ph, pw, s), TOL, f"conv bwd-data {case}")
    e3 = assert_close(dw.asnumpy(), O.conv2d_grad_filter(x, dy, w.shape, ph, pw, s), TOL, f"conv bwd-filter {case}")
    assert max(e1, e2, e3) < 1e-4


def test_input_beyond_two_gib():
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    N, C, H, W = 36, 16, 1000, 1000                     # 2.30 GB per tensor
    rng = np.random.RandomState(8)
    base = rng.standard_normal((C, H, W)).astype(np.float32)
    x = np.empty((N, C, H, W), np.float32)
    for i in range(N):                                  # every image different, cheaply
        np.multiply(np.roll(base, 37 * i, axis=2), 1.0 + i / 64.0, out=x[i])
    gx = ndarray.array(x, ctx)
    y = ndarray.empty((N, C, H, W), ctx)

    # 1. delta filters: output channel o is input channel perm[o], exactly, in all 576 M positions
    perm = rng.permutation(C)
    wd = np.zeros((C, C, 3, 3), np.float32)
    wd[np.arange(C), perm, 1, 1] = 1.0
    gwd = ndarray.array(wd, ctx)
    L.CuDNN_conv2d(gx, gwd, y, 1, 1, 1)
    got = y.asnumpy()
    for i in range(N):
        assert np.array_equal(got[i], x[i][perm]), "forward, image %d" % i
    # ... and its adjoint: dx channel perm[o] is dy channel o
    dx = ndarray.empty((N, C, H, W), ctx)
    L.CuDNN_conv2d_gradient_of_data(gwd, gx, dx, 1, 1, 1)
    got = dx.asnumpy()
    inv = np.argsort(perm)
    for i in range(N):
        assert np.array_equal(got[i], x[i][inv]), "backward-data, image %d" % i
    del got

    # 2. a dense filter: the images on both sides of every run boundary equal the per-image result
    w = (rng.standard_normal((C, C, 3, 3)) / 12.0).astype(np.float32)
    gw = ndarray.array(w, ctx)
    L.CuDNN_conv2d(gx, gw, y, 1, 1, 1)
    L.CuDNN_conv2d_gradient_of_data(gw, gx, dx, 1, 1, 1)
    one_y, one_dx = ndarray.empty((1, C, H, W), ctx), ndarray.empty((1, C, H, W), ctx)
    for i in (0, 1, 17, 18, 34, 35):
        xi = ndarray.slice_for_micro_tensor(gx, i, N, "batch")
        L.CuDNN_conv2d(xi, gw, one_y, 1, 1, 1)
        L.CuDNN_conv2d_gradient_of_data(gw, xi, one_dx, 1, 1, 1)
        assert_close(ndarray.slice_for_micro_tensor(y, i, N, "batch").asnumpy(), one_y.asnumpy(), 1e-5, "forward %d" % i)
        assert_close(ndarray.slice_for_micro_tensor(dx, i, N, "batch").asnumpy(), one_dx.asnumpy(), 1e-5,
                     "backward-data %d" % i)

    # 3. filter gradient of (x, dy = y): equals the sum of the 36 per-image gradients
    dw = ndarray.empty((C, C, 3, 3), ctx)
    L.CuDNN_conv2d_gradient_of_filter(gx, y, dw, 1, 1, 1)
    total = np.zeros((C, C, 3, 3), np.float64)
    one_dw = ndarray.empty((C, C, 3, 3), ctx)
    for i in range(N):
        L.CuDNN_conv2d_gradient_of_filter(ndarray.slice_for_micro_tensor(gx, i, N, "batch"),
                                          ndarray.slice_for_micro_tensor(y, i, N, "batch"), one_dw, 1, 1, 1)
        total += one_dw.asnumpy()
    assert_close(dw.asnumpy(), total, 1e-4, "filter gradient")
