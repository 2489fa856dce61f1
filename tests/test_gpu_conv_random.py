"""A seeded sweep of random small convolution geometries through all three passes against the CPU
oracle.  The dispatcher picks among many kernels by shape (thin first layer, tap-major kernels
with and without padded image tails, stride phases, the few-columns filter gradient, the gather
engine); the sweep draws channel counts around the multiples of 16 those choices hinge on, odd
image sizes, filters from 1x1 to 7x7 (square or not), paddings up to the filter size and strides
1-3, so every branch meets shapes nobody wrote down by hand."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 2e-3


def _cases(seed, count):
    rng = np.random.RandomState(seed)
    chans = [1, 2, 3, 5, 8, 15, 16, 17, 24, 31, 32, 33, 48, 64, 65, 80, 130]
    out = []
    while len(out) < count:
        kH, kW = rng.choice([1, 2, 3, 5, 7]), rng.choice([1, 2, 3, 5, 7])
        if rng.rand() < 0.6:
            kW = kH
        s = int(rng.choice([1, 1, 1, 2, 2, 3]))
        ph, pw = int(rng.randint(0, kH // 2 + 2)), int(rng.randint(0, kW // 2 + 2))
        H, W = int(rng.randint(1, 26)), int(rng.randint(1, 26))
        if H + 2 * ph < kH or W + 2 * pw < kW:
            continue
        N = int(rng.choice([1, 2, 3, 5]))
        C, Oc = int(rng.choice(chans)), int(rng.choice(chans))
        if N * C * H * W * Oc * kH * kW > 6e8:       # keep the float64 oracle quick
            continue
        out.append((N, C, H, W, Oc, int(kH), int(kW), ph, pw, s))
    return out


@pytest.mark.parametrize("case", _cases(2024, 300))
def test_random_geometry(case):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    N, C, H, W, Oc, kH, kW, ph, pw, s = case
    rng = np.random.RandomState(abs(hash(case)) % (2 ** 31))
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, kH, kW)) / np.sqrt(C * kH * kW)).astype(np.float32)
    ref_y = O.conv2d(x, w, ph, pw, s)
    dy = rng.normal(size=ref_y.shape).astype(np.float32)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    y, dx, dw = ndarray.empty(ref_y.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
    L.CuDNN_conv2d(gx, gw, y, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, ph, pw, s)
    e1 = assert_close(y.asnumpy(), ref_y, TOL, f"conv fwd {case}")
    e2 = assert_close(dx.asnumpy(), O.conv2d_grad_data(w, dy, x.shape, ph, pw, s), TOL, f"conv bwd-data {case}")
    e3 = assert_close(dw.asnumpy(), O.conv2d_grad_filter(x, dy, w.shape, ph, pw, s), TOL, f"conv bwd-filter {case}")
    assert max(e1, e2, e3) < 1e-4


def _winograd_cases(seed, count):
    """3x3 / stride 1 / pad 1 layers around the shapes the Winograd forms branch on: channel counts that are and are
    not multiples of 16 / 64, planes that are and are not multiples of 4 (the one-kernel forms take only those),
    one image to sixteen."""
    rng = np.random.RandomState(seed)
    chans = [16, 32, 48, 64, 64, 64, 80, 128, 128, 192, 256]
    sides = [4, 8, 12, 16, 20, 24, 28, 32, 36, 40, 44, 56, 60, 64, 7, 13, 17, 30]
    out = []
    while len(out) < count:
        C, Oc = int(rng.choice(chans)), int(rng.choice(chans))
        H, W = int(rng.choice(sides)), int(rng.choice(sides))
        N = int(rng.choice([1, 2, 3, 4, 5, 8, 16]))
        if N * C * H * W * Oc * 9 > 1.2e9:           # keep the float64 oracle quick
            continue
        out.append((N, C, H, W, Oc, 3, 3, 1, 1, 1))
    return out


@pytest.mark.parametrize("case", _winograd_cases(77, 120))
def test_random_geometry_through_the_winograd_routine(case, monkeypatch):
    """The same three passes with every layer forced through the Winograd routine (whose forms then choose
    themselves by shape: one kernel, three kernels, runs of tiles or rectangles of them).  Its rounding error is
    ten times a direct sum's: 2e-5 of the output's magnitude at most over 2 600 such draws, held to 1e-4 here."""
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    N, C, H, W, Oc, kH, kW, ph, pw, s = case
    rng = np.random.RandomState(abs(hash(case)) % (2 ** 31))
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, kH, kW)) / np.sqrt(C * kH * kW)).astype(np.float32)
    ref_y = O.conv2d(x, w, ph, pw, s)
    dy = rng.normal(size=ref_y.shape).astype(np.float32)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    y, dx, dw = ndarray.empty(ref_y.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
    L.CuDNN_conv2d(gx, gw, y, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, ph, pw, s)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, ph, pw, s)
    e1 = assert_close(y.asnumpy(), ref_y, TOL, f"conv fwd {case}")
    e2 = assert_close(dx.asnumpy(), O.conv2d_grad_data(w, dy, x.shape, ph, pw, s), TOL, f"conv bwd-data {case}")
    e3 = assert_close(dw.asnumpy(), O.conv2d_grad_filter(x, dy, w.shape, ph, pw, s), TOL, f"conv bwd-filter {case}")
    assert max(e1, e2, e3) < 1e-4
