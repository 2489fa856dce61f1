"""The opt-in split-bf16 products of the Winograd routine's GEMMs and of the matrix products (TSplit_SplitBf16),
through the C ABI.

Bars: with the switch on, the three convolutions of wide 3x3 layers meet the float64 oracle within the
convolution tolerance (2e-3 max relative error, and below 1e-4 as the fp32 path does), their error against
the oracle is no larger than 1.5 times the fp32 path's on the same inputs (the six bf16 products leave out
less than the rounding of an fp32 multiplication), layers the switch does not cover give the same bits as
before, and a network with such layers still tracks the oracle's training run."""
import numpy as np
import pytest

from oracle import nets, ops as O
from util import assert_close, max_rel_err

pytestmark = pytest.mark.gpu
TOL = 2e-3

# N, C, H, W, O: 3x3 / stride 1 / pad 1 layers with more than 64 channels on both sides
CASES = [
    (4, 128, 28, 28, 128),     # whole tiles
    (3, 80, 30, 26, 144),      # ragged rows and columns, five k-steps, planes the tiling overhangs
    (2, 72, 18, 22, 136),      # channel counts that only the filter gradient takes through the routine
    (2, 256, 14, 14, 192),     # two row tiles, few columns
    (16, 128, 56, 56, 256),    # the filter gradient cut into ranges, several rounds of the persistent grid
]


@pytest.fixture
def split():
    from tsplit_amd import gpu_links as L
    was = L.split_bf16(False)
    yield L
    L.split_bf16(was)


def _three_passes(L, nd, ctx, x, w, dy):
    gx, gw, gdy = nd.array(x, ctx), nd.array(w, ctx), nd.array(dy, ctx)
    y, dx, dw = nd.empty(dy.shape, ctx), nd.empty(x.shape, ctx), nd.empty(w.shape, ctx)
    L.CuDNN_conv2d(gx, gw, y, 1, 1, 1)
    L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, 1, 1, 1)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, 1, 1, 1)
    return y.asnumpy(), dx.asnumpy(), dw.asnumpy()


@pytest.mark.parametrize("case", CASES)
def test_split_products_meet_the_oracle_as_closely_as_fp32(case, rng, split, monkeypatch):
    from tsplit_amd import ndarray as nd
    L, ctx = split, nd.gpu(0)
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    N, C, H, W, Oc = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, 3, 3)) / np.sqrt(C * 9)).astype(np.float32)
    dy = rng.normal(size=(N, Oc, H, W)).astype(np.float32)
    L.winograd_gemm_timing(True)
    plain = _three_passes(L, nd, ctx, x, w, dy)
    assert L.winograd_gemm_times(kind=3)[0] == 0 and L.winograd_gemm_times(kind=4)[0] == 0
    assert L.split_bf16(True) is False
    got = _three_passes(L, nd, ctx, x, w, dy)
    # the split kernels ran: forward and data gradient (where the summed channels are a multiple of 16, else
    # those passes take the direct kernels) and the filter gradient
    assert L.winograd_gemm_times(kind=3)[0] == (C % 16 == 0) + (Oc % 16 == 0) and L.winograd_gemm_times(kind=4)[0] == 1
    L.winograd_gemm_timing(False)
    if N * C * H * W <= 1 << 21:
        refs = (O.conv2d(x, w, 1, 1, 1), O.conv2d_grad_data(w, dy, x.shape, 1, 1, 1), O.conv2d_grad_filter(x, dy, w.shape, 1, 1, 1))
    else:   # too large for the oracle's loops: compared with the fp32 path below
        refs = None
    for i, name in enumerate(("forward", "data gradient", "filter gradient")):
        if refs is not None:
            e_split = assert_close(got[i], refs[i], TOL, f"split {name} {case}")
            e_plain = max_rel_err(plain[i], refs[i])
            assert e_split < 1e-4
            assert e_split <= 1.5 * e_plain + 1e-7, (name, e_split, e_plain)
        else:
            # both paths compute the same sums and round differently (each lies within 2e-5 of the exact
            # result, the Winograd transforms' share): they agree far inside the tolerance
            assert_close(got[i], plain[i], 5e-5, f"split against fp32 {name} {case}")


def test_layers_outside_the_switch_keep_their_bits(rng, split, monkeypatch):
    """64 channels on one side (64 x 256 tiles, narrow filter-gradient tiles), a depth that is not a multiple of
    8, and the direct kernels are untouched by the switch."""
    from tsplit_amd import ndarray as nd
    L, ctx = split, nd.gpu(0)
    for case, forced in [((4, 64, 28, 28, 64), "1"), ((4, 64, 28, 28, 128), "1"), ((2, 128, 20, 20, 64), "1"),
                         ((2, 128, 14, 14, 128), "0")]:
        monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", forced)
        N, C, H, W, Oc = case
        x = rng.normal(size=(N, C, H, W)).astype(np.float32)
        w = (rng.normal(size=(Oc, C, 3, 3)) / np.sqrt(C * 9)).astype(np.float32)
        dy = rng.normal(size=(N, Oc, H, W)).astype(np.float32)
        L.split_bf16(False)
        plain = _three_passes(L, nd, ctx, x, w, dy)
        L.split_bf16(True)
        got = _three_passes(L, nd, ctx, x, w, dy)
        L.split_bf16(False)
        for i, name in enumerate(("forward", "data gradient", "filter gradient")):
            covered = forced == "1" and ((i == 0 and Oc > 64) or (i == 1 and C > 64) or (i == 2 and C > 64 and Oc > 64))
            if covered:
                assert_close(got[i], plain[i], 5e-5, f"{name} {case}")
            else:
                np.testing.assert_array_equal(got[i], plain[i], err_msg=f"{name} {case}")


def test_operands_with_extreme_exponents(split, monkeypatch):
    """Terms of the split keep fp32's exponent range: activations of 1e-30 and 1e+30 with filters of 1e-3."""
    from tsplit_amd import ndarray as nd
    L, ctx = split, nd.gpu(0)
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    rng = np.random.RandomState(3)
    x = rng.normal(size=(2, 128, 12, 12)).astype(np.float32)
    w = (rng.normal(size=(128, 128, 3, 3)) * 1e-3).astype(np.float32)
    L.split_bf16(True)
    for scale in (1e-30, 1.0, 1e30):
        xs = (x * np.float32(scale)).astype(np.float32)
        y = nd.empty(x.shape, ctx)
        L.CuDNN_conv2d(nd.array(xs, ctx), nd.array(w, ctx), y, 1, 1, 1)
        assert_close(y.asnumpy() / np.float32(scale), O.conv2d(x, w, 1, 1, 1), 1e-4, f"scale {scale}")


MATMULS = [
    # M, K, N
    (64, 4096, 1000),      # a fully-connected layer at batch 64: one row tile half empty, the depth cut into ranges
    (200, 72, 300),        # ragged rows and columns, a depth that is a multiple of 4 only
    (256, 512, 2048),      # whole tiles
    (130, 20, 70),         # one full and one partial k-step
]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("shape", MATMULS)
def test_matrix_product_with_split_terms(shape, ta, tb, rng, split):
    """DLGpuMatrixMultiply in its four transpose forms: against float64 no further off than 1.5 times the fp32
    matrix instruction's own error (relative to the sum of the products' magnitudes), inside the 2e-3 tolerance."""
    from tsplit_amd import ndarray as nd
    L, ctx = split, nd.gpu(0)
    M, K, N = shape
    a = rng.normal(size=(K, M) if ta else (M, K)).astype(np.float32)
    b = rng.normal(size=(N, K) if tb else (K, N)).astype(np.float32)
    a64, b64 = (a.T if ta else a).astype(np.float64), (b.T if tb else b).astype(np.float64)
    ref, mag = a64 @ b64, np.abs(a64) @ np.abs(b64)
    ga, gb = nd.array(a, ctx), nd.array(b, ctx)
    outs = []
    for on in (False, True):
        L.split_bf16(on)
        c = nd.empty((M, N), ctx)
        L.matrix_multiply(ga, ta, gb, tb, c)
        outs.append(c.asnumpy())
    L.split_bf16(False)
    e_plain, e_split = [(np.abs(o - ref) / mag).max() for o in outs]
    assert_close(outs[1], ref, TOL, f"matmul {shape} ta={ta} tb={tb}")
    assert e_split <= 1.5 * e_plain + 1e-8, (e_split, e_plain)
    assert not np.array_equal(outs[0], outs[1])      # the split kernel did run


def test_matrix_product_outside_the_switch_keeps_its_bits(rng, split):
    """A depth that is not a multiple of 4 stays on the fp32 kernels."""
    from tsplit_amd import ndarray as nd
    L, ctx = split, nd.gpu(0)
    a, b = rng.normal(size=(70, 30)).astype(np.float32), rng.normal(size=(30, 90)).astype(np.float32)
    ga, gb = nd.array(a, ctx), nd.array(b, ctx)
    outs = []
    for on in (False, True):
        L.split_bf16(on)
        c = nd.empty((70, 90), ctx)
        L.matrix_multiply(ga, False, gb, False, c)
        outs.append(c.asnumpy())
    L.split_bf16(False)
    np.testing.assert_array_equal(outs[0], outs[1])


def _onehot(lab, n):
    out = np.zeros((len(lab), n), np.float32)
    out[np.arange(len(lab)), lab] = 1
    return out


def test_training_with_split_products_tracks_oracle(split, monkeypatch):
    """Six momentum steps of a small net whose 3x3 layers have 96 and 128 channels, every wide layer through the
    Winograd routine with split products, against the oracle's run (loss 1e-3, parameters 2e-3)."""
    from tsplit_amd import ndarray, trainer
    L = split
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    rng = np.random.RandomState(11)
    spec = [("conv", "c1", 3, 96, 3, 1, 1), ("bn", "c1_bn", 96), ("relu",),
            ("conv", "c2", 96, 128, 3, 1, 1), ("bn", "c2_bn", 128), ("relu",), ("maxpool", 2, 0, 2),
            ("conv", "c3", 128, 128, 3, 1, 1), ("bn", "c3_bn", 128), ("relu",), ("maxpool", 2, 0, 2),
            ("flatten",), ("fc", "f1", 128 * 4 * 4, 64), ("fc", "f2", 64, 10)]
    X = rng.normal(size=(8, 3, 16, 16)).astype(np.float32)
    Y = _onehot(rng.randint(0, 10, 8), 10)
    params = trainer.init_params(spec, seed=5)
    ref_losses, ref_params = nets.train(spec, params, X, Y, steps=6, lr=0.05, momentum=0.9)
    ctx = ndarray.gpu(0)
    L.split_bf16(True)
    L.winograd_gemm_timing(True)
    t = trainer.Trainer(spec, params, X.shape, 10, ctx, optimizer=("momentum", 0.05, 0.9))
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for _ in range(6):
        t.step(gx, gy)
        losses.append(t.loss_value())
    assert L.winograd_gemm_times(kind=3)[0] > 0 and L.winograd_gemm_times(kind=4)[0] > 0
    L.winograd_gemm_timing(False)
    rel = np.max(np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses))
    assert rel <= 1e-3, (rel, losses, ref_losses)
    for k in params:
        assert_close(t.params[k].asnumpy(), ref_params[k], 2e-3, k)
