"""GPU parity of the three convolutions (implicit GEMM on fp32 MFMA; Winograd F(4x4, 3x3) for wide
3x3 layers) against the CPU oracle, through both symbol families.  Tolerance 2e-3 max relative
error; measured errors are ~1e-6 (direct) and below 2e-5 (Winograd)."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 2e-3

CASES = [
    # N, C, H, W, O, kH, kW, ph, pw, stride
    (2, 3, 6, 6, 4, 3, 3, 1, 1, 1),
    (1, 2, 7, 7, 3, 3, 3, 1, 1, 2),
    (2, 2, 8, 8, 3, 3, 3, 1, 1, 2),        # stride 2 with flooring
    (1, 3, 9, 9, 2, 7, 7, 3, 3, 2),        # ResNet stem class
    (1, 2, 5, 8, 3, 1, 7, 0, 3, 1),        # 1x7, asymmetric padding
    (1, 2, 8, 5, 3, 7, 1, 3, 0, 1),        # 7x1
    (2, 4, 5, 5, 3, 1, 1, 0, 0, 1),        # 1x1
    (1, 2, 6, 6, 2, 3, 3, 0, 0, 1),        # valid
    (2, 3, 32, 32, 64, 3, 3, 1, 1, 1),     # VGG conv1_1 class: K = 27, 64x256 tiles
    (2, 64, 28, 28, 64, 3, 3, 1, 1, 1),    # 64 -> 64
    (4, 64, 56, 56, 128, 3, 3, 1, 1, 1),   # 128x128 tiles
    (2, 128, 14, 14, 256, 3, 3, 1, 1, 1),  # two M tiles, N = 392 (ragged)
    (3, 20, 17, 13, 70, 3, 3, 1, 1, 1),    # everything ragged
    (2, 16, 15, 15, 24, 3, 3, 1, 1, 2),    # stride 2, odd output 8x8
    (2, 8, 7, 7, 40, 1, 1, 0, 0, 1),       # oH*oW = 49: not a multiple of 4
    (2, 6, 12, 12, 130, 5, 5, 2, 2, 1),
    # forward / backward-data cut the k-steps of all tiles into equal ranges, one per resident
    # block; the pieces of a cut tile are assembled by a second kernel
    (25, 16, 64, 64, 128, 3, 3, 1, 1, 1),  # 800 tiles of 128x128 (forward)
    (13, 16, 128, 128, 16, 3, 3, 1, 1, 1), # 832 tiles of 64x256 (forward and backward-data)
    # fewer tiles than resident blocks: every tile is cut into many pieces
    (8, 512, 14, 14, 256, 3, 3, 1, 1, 1),  # 26 tiles of 128x128, 288 k-steps each
    (8, 512, 28, 28, 64, 3, 3, 1, 1, 1),   # forward on 64x256 tiles
    (8, 64, 28, 28, 512, 3, 3, 1, 1, 1),   # backward-data on 64x256 tiles
    # strided convolutions: backward-data runs one GEMM per stride phase
    (2, 32, 14, 14, 48, 1, 1, 0, 0, 2),    # 1x1 stride 2 (ResNet shortcut): three of four phases are zero
    (2, 24, 15, 15, 40, 3, 3, 1, 1, 2),    # 3x3 stride 2 pad 1, odd input
    (2, 16, 17, 17, 20, 3, 3, 0, 0, 2),    # 3x3 stride 2 valid (Inception reductions)
    (1, 8, 23, 19, 12, 7, 7, 3, 3, 2),     # 7x7 stride 2 pad 3 (ResNet stem), non-square
    (2, 8, 20, 20, 12, 5, 5, 2, 2, 3),     # stride 3
    (1, 70, 12, 12, 130, 3, 3, 1, 1, 2),   # 128x128 tiles, ragged
    (1, 4, 9, 9, 6, 2, 2, 0, 0, 3),        # stride larger than the filter: some inputs get no gradient
    # the same with output channels in multiples of 16: the phases run on the buffer-load kernel
    (2, 24, 15, 15, 48, 3, 3, 1, 1, 2),
    (2, 16, 17, 17, 32, 3, 3, 0, 0, 2),
    (1, 8, 23, 19, 16, 7, 7, 3, 3, 2),
    (2, 8, 20, 20, 16, 5, 5, 2, 2, 3),
    (1, 70, 12, 12, 144, 3, 3, 1, 1, 2),
    (1, 4, 9, 9, 16, 2, 2, 0, 0, 3),
    (8, 64, 56, 56, 128, 3, 3, 1, 1, 2),   # ResNet stage transition: tiles cut between blocks
    (4, 256, 28, 28, 512, 1, 1, 0, 0, 2),  # ResNet shortcut, 128x128 tiles in two rows
    # at most 32 filter columns (C*kH*kW): backward-filter takes the few-columns kernel
    (4, 3, 64, 64, 64, 3, 3, 1, 1, 1),     # several K slices, folded
    (3, 1, 19, 23, 100, 5, 5, 2, 2, 1),    # 25 columns, two row tiles, ragged K (oH*oW odd)
    (2, 2, 20, 20, 33, 4, 4, 1, 1, 2),     # exactly 32 columns, stride 2
    (1, 3, 5, 5, 7, 3, 3, 1, 1, 1),        # K = 25: one partial step
    # "same" stride-1 filters with H*W a multiple of 4 but not of 16: the tap-major backward-filter
    # kernel pads each image's positions to a multiple of 16
    (3, 16, 6, 6, 20, 3, 3, 1, 1, 1),      # 36 positions, image rows shorter than one k-step
    (2, 16, 2, 2, 8, 3, 3, 1, 1, 1),       # 4 positions
    (2, 32, 10, 14, 24, 1, 7, 0, 3, 1),    # 140 positions, 1x7 filter
    (5, 48, 14, 14, 72, 3, 3, 1, 1, 1),    # 196 positions, odd image count
    # ... and not a multiple of 4: the 16-byte gradient words start on 4-byte boundaries and the
    # last word of an image straddles into the next row
    (2, 16, 7, 7, 24, 3, 3, 1, 1, 1),      # 49 positions
    (3, 32, 17, 17, 40, 1, 7, 0, 3, 1),    # 289 positions, 1x7
    (2, 16, 5, 5, 8, 1, 1, 0, 0, 1),       # 25 positions, 1x1
    (2, 16, 35, 35, 20, 3, 3, 1, 1, 1),    # 1225 positions
    (3, 16, 3, 5, 136, 3, 3, 1, 1, 1),     # 15 positions: less than one k-step, two row tiles
    # strided and "valid" filters with input channels in multiples of 16: the same backward-filter
    # kernel with every thread tracking the (row, column) of its output position
    (3, 32, 21, 21, 32, 3, 3, 0, 0, 1),    # 3x3 valid (Inception stem): 361 positions
    (2, 16, 32, 32, 24, 3, 3, 0, 0, 1),    # 900 positions, a multiple of 4 only
    (2, 16, 18, 18, 24, 3, 3, 0, 0, 1),    # 256 positions: whole k-steps
    (5, 16, 9, 9, 40, 3, 3, 1, 1, 2),      # 25 output positions per image, stride 2
    (2, 48, 16, 16, 136, 1, 1, 0, 0, 2),   # 1x1 stride 2: 64 positions, two row tiles
    (2, 16, 23, 19, 24, 7, 7, 3, 3, 2),    # 7x7 stride 2, non-square
    (2, 16, 20, 20, 12, 5, 5, 2, 2, 3),    # stride 3
    (3, 16, 6, 40, 8, 1, 7, 0, 0, 1),      # 1x7 valid: output narrower than the input
    (2, 32, 5, 5, 16, 5, 5, 0, 0, 1),      # one output position per image
    (1, 16, 9, 9, 16, 2, 2, 0, 0, 3),      # stride larger than the filter
]


def _run(case, family, rng):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    N, C, H, W, Oc, kH, kW, ph, pw, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = (rng.normal(size=(Oc, C, kH, kW)) / np.sqrt(C * kH * kW)).astype(np.float32)
    ref_y = O.conv2d(x, w, ph, pw, s)
    dy = rng.normal(size=ref_y.shape).astype(np.float32)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    y, dx, dw = ndarray.empty(ref_y.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
    if family == "cudnn":
        L.CuDNN_conv2d(gx, gw, y, ph, pw, s)
        L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, ph, pw, s)
        L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, ph, pw, s)
    else:
        ws = ndarray.empty((1,), ctx)          # the im2col workspaces are accepted and unused
        L.conv2d(gx, gw, y, ws, ph, s)
        L.conv2d_gradient_of_data(gw, gdy, dx, ws, ph, s)
        L.conv2d_gradient_of_filter(gx, gdy, dw, ws, ws, ph, s)
    e1 = assert_close(y.asnumpy(), ref_y, TOL, f"conv fwd {case}")
    e2 = assert_close(dx.asnumpy(), O.conv2d_grad_data(w, dy, x.shape, ph, pw, s), TOL, f"conv bwd-data {case}")
    e3 = assert_close(dw.asnumpy(), O.conv2d_grad_filter(x, dy, w.shape, ph, pw, s), TOL, f"conv bwd-filter {case}")
    assert max(e1, e2, e3) < 1e-4


@pytest.mark.parametrize("case", CASES)
def test_conv_cudnn_family(case, rng):
    _run(case, "cudnn", rng)


@pytest.mark.parametrize("raw", ["0", "1"])
@pytest.mark.parametrize("case", [c for c in CASES if c[9] == 1 and c[4] % 16 == 0])
def test_conv_backward_data_with_and_without_filter_relay(case, raw, rng, monkeypatch):
    """Stride-1 backward-data with output channels in multiples of 16 has two kernels: one reads a
    re-laid copy of the filter, one (chosen for small layers) the filter where it lies.  Both run on
    every such shape."""
    monkeypatch.setenv("TSPLIT_CONV_RAW", raw)
    _run(case, "cudnn", rng)


WINOGRAD_CASES = [c for c in CASES if c[5:] == (3, 3, 1, 1, 1) and c[1] % 16 == 0 and c[4] % 16 == 0] + [
    (4, 128, 28, 28, 128, 3, 3, 1, 1, 1),   # whole 4x4 tiles, rows stored as quads
    (2, 256, 14, 14, 144, 3, 3, 1, 1, 1),   # 14 = 3.5 tiles: the last tile row and column hang over the edge
    (3, 32, 13, 17, 48, 3, 3, 1, 1, 1),     # odd, non-square planes
    (2, 16, 5, 3, 16, 3, 3, 1, 1, 1),       # a plane narrower than one tile
    (1, 16, 1, 1, 16, 3, 3, 1, 1, 1),       # one pixel: only the filter's centre counts
    (3, 16, 40, 72, 32, 3, 3, 1, 1, 1),     # 18 tiles per row: tile rows do not line up with the 64 lanes of a wave
    (2, 16, 300, 260, 16, 3, 3, 1, 1, 1),   # tile rows longer than a wave
    (70, 32, 8, 8, 48, 3, 3, 1, 1, 1),      # 280 tiles: the tile count padded to a multiple of 4 and of 128
]


@pytest.mark.parametrize("winograd", ["0", "1"])
@pytest.mark.parametrize("case", WINOGRAD_CASES)
def test_conv_3x3_direct_and_winograd(case, winograd, rng, monkeypatch):
    """3x3 / stride 1 / pad 1 layers have two routines for each of the three passes: the direct
    implicit GEMM and Winograd F(4x4, 3x3) (chosen for wide layers).  Both run on every
    such shape; the Winograd transforms cost about a digit (errors of a few 1e-6 of the output's
    magnitude against ~1e-7), far inside the 2e-3 bar, and `_run` holds both to 1e-4."""
    from tsplit_amd import gpu_links as L
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", winograd)
    N, C, H, W, Oc = case[:5]
    assert L.conv_takes_winograd(N, C, Oc, H, W) == (winograd == "1")
    assert L.conv_takes_winograd(N, C, Oc, H, W, data_gradient=True) == (winograd == "1")
    assert L.conv_takes_winograd(N, C, Oc, H, W, filter_gradient=True) == (winograd == "1")
    _run(case, "cudnn", rng)


def test_conv_winograd_choice(monkeypatch):
    """Left to itself the library takes Winograd for wide 3x3 / stride 1 / pad 1 layers with enough
    tiles, and never for another filter, stride or padding, whatever the environment says."""
    from tsplit_amd import gpu_links as L
    monkeypatch.delenv("TSPLIT_CONV_WINOGRAD", raising=False)
    assert L.conv_takes_winograd(64, 256, 256, 56, 56) and L.conv_takes_winograd(64, 256, 256, 56, 56, data_gradient=True)
    assert L.conv_takes_winograd(16, 64, 128, 112, 112) and L.conv_takes_winograd(64, 512, 512, 14, 14)
    assert L.conv_takes_winograd(64, 256, 256, 56, 56, filter_gradient=True)
    assert L.conv_takes_winograd(16, 64, 128, 112, 112, filter_gradient=True)
    assert L.conv_takes_winograd(16, 64, 64, 224, 224, filter_gradient=True)
    assert not L.conv_takes_winograd(16, 32, 64, 224, 224, filter_gradient=True)
    # 64 channels on both sides are enough in every pass (tiles as wide as the produced channels)
    assert L.conv_takes_winograd(64, 64, 64, 224, 224) and L.conv_takes_winograd(16, 64, 64, 224, 224, data_gradient=True)
    assert not L.conv_takes_winograd(64, 32, 64, 224, 224) and not L.conv_takes_winograd(64, 64, 48, 224, 224)   # too narrow
    assert not L.conv_takes_winograd(2, 256, 256, 14, 14)            # too few tiles
    assert not L.conv_takes_winograd(64, 3, 64, 224, 224)
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    assert L.conv_takes_winograd(2, 16, 16, 5, 5)
    assert not L.conv_takes_winograd(2, 24, 16, 5, 5)                # channels summed over must be a multiple of 16
    assert L.conv_takes_winograd(2, 24, 16, 5, 5, data_gradient=True)
    assert L.conv_takes_winograd(2, 24, 20, 5, 5, filter_gradient=True)   # any channel counts
    assert not L.conv_takes_winograd(2, 3, 20, 5, 5, filter_gradient=True)  # at most 32 filter columns: the narrow kernel
    for kernel, pad, stride in ((3, 1, 2), (3, 0, 1), (1, 0, 1), (5, 2, 1)):
        assert not L.conv_takes_winograd(64, 256, 256, 56, 56, kernel, pad, stride)
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "0")
    assert not L.conv_takes_winograd(64, 256, 256, 56, 56)


def test_conv_winograd_is_per_image_and_repeatable(rng, monkeypatch):
    """Tiles never span images and every GEMM sums the channels in one fixed order: a batch run as 4
    micro-tensors, in runs of a few images (a small scratch allowance) or twice gives the same bits."""
    from tsplit_amd import gpu_links as L, ndarray
    monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", "1")
    ctx = ndarray.gpu(0)
    x = rng.normal(size=(8, 32, 20, 24)).astype(np.float32)
    w = rng.normal(size=(48, 32, 3, 3)).astype(np.float32)
    dy = rng.normal(size=(8, 48, 20, 24)).astype(np.float32)
    gx, gw, gdy = ndarray.array(x, ctx), ndarray.array(w, ctx), ndarray.array(dy, ctx)
    dws = []
    for _ in range(2):                     # the filter gradient sums over images: repeatable, not splittable
        dw = ndarray.empty(w.shape, ctx)
        L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, 1, 1, 1)
        dws.append(dw.asnumpy())
    np.testing.assert_array_equal(dws[0], dws[1])

    def both(split):
        y, dx = ndarray.empty(dy.shape, ctx), ndarray.empty(x.shape, ctx)
        if split:
            for a in (gx, gdy, y, dx):
                a.split_tensor(4)
            for i in range(4):
                L.CuDNN_conv2d(gx.sTensor[i], gw, y.sTensor[i], 1, 1, 1)
                L.CuDNN_conv2d_gradient_of_data(gw, gdy.sTensor[i], dx.sTensor[i], 1, 1, 1)
        else:
            L.CuDNN_conv2d(gx, gw, y, 1, 1, 1)
            L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, 1, 1, 1)
        return y.asnumpy(), dx.asnumpy()

    whole = both(False)
    again = both(False)
    monkeypatch.setenv("TSPLIT_WINOGRAD_RUN_MIB", "1")     # 3 images per run
    runs = both(False)
    monkeypatch.delenv("TSPLIT_WINOGRAD_RUN_MIB")
    parts = both(True)
    for other in (again, runs, parts):
        np.testing.assert_array_equal(whole[0], other[0])
        np.testing.assert_array_equal(whole[1], other[1])


@pytest.mark.parametrize("shape", [(4, 64, 128, 128, 128),      # 4096 tiles, rows of 32 tiles: whole steps of 8
                                   (6, 128, 64, 120, 92),       # 4140 tiles, rows of 23: steps wrap rows and images, ragged end
                                   (5, 128, 128, 116, 116),     # 4205 tiles, four band pairs
                                   (300, 64, 64, 16, 16)])      # 4800 tiles, rows of 4: a step of 8 covers two rows of tiles
def test_conv_winograd_filter_gradient_in_one_kernel(shape, rng):
    """Layers with at most 128 channels and at least 4096 tiles take the filter gradient that transforms both
    tensors on the way into LDS (wino_fgrad_fused.h).  Channel blocks of 8 x 8 filters (a filter's gradient depends
    on its two channels only), chosen inside bands, across the band boundary and at the end, against the oracle;
    the whole result against the direct kernels; twice for the same bits."""
    from tsplit_amd import gpu_links as L, ndarray
    import os
    N, C, Oc, H, W = shape
    ctx = ndarray.gpu(0)
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    dy = rng.normal(size=(N, Oc, H, W)).astype(np.float32)
    gx, gdy = ndarray.array(x, ctx), ndarray.array(dy, ctx)
    assert L.conv_takes_winograd(N, C, Oc, H, W, filter_gradient=True)
    L.winograd_gemm_timing(True, kind=6)
    got = []
    for _ in range(2):
        dw = ndarray.empty((Oc, C, 3, 3), ctx)
        L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, 1, 1, 1)
        got.append(dw.asnumpy())
    launches = L.winograd_gemm_times(kind=6)[0]
    L.winograd_gemm_timing(False)
    assert launches == 2, "the one-kernel filter gradient did not run"
    np.testing.assert_array_equal(got[0], got[1])
    scale = np.max(np.abs(got[0]))
    for o0, c0 in ((0, 0), (Oc - 8, C - 8), (min(60, Oc - 8), min(60, C - 8)), (17, C - 8)):
        ref = O.conv2d_grad_filter(x[:, c0:c0 + 8], dy[:, o0:o0 + 8], (8, 8, 3, 3), 1, 1, 1)
        err = np.max(np.abs(got[0][o0:o0 + 8, c0:c0 + 8] - ref)) / scale
        assert err <= 1e-4, (o0, c0, err)
    os.environ["TSPLIT_CONV_WINOGRAD"] = "0"
    try:
        direct = ndarray.empty((Oc, C, 3, 3), ctx)
        L.CuDNN_conv2d_gradient_of_filter(gx, gdy, direct, 1, 1, 1)
        assert_close(got[0], direct.asnumpy(), 1e-4, f"one-kernel Winograd filter gradient vs direct {shape}")
    finally:
        del os.environ["TSPLIT_CONV_WINOGRAD"]


@pytest.mark.parametrize("case", [c for c in CASES if c[7] == c[8]][:8])
def test_conv_plain_family(case, rng):
    _run(case, "plain", rng)


def test_conv_micro_tensor_split_is_bit_identical(rng):
    """Conv is per-sample: running it on 4 batch views gives exactly the unsplit result."""
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    x = rng.normal(size=(8, 16, 20, 20)).astype(np.float32)
    w = rng.normal(size=(32, 16, 3, 3)).astype(np.float32)
    gx, gw = ndarray.array(x, ctx), ndarray.array(w, ctx)
    whole, parts = ndarray.empty((8, 32, 20, 20), ctx), ndarray.empty((8, 32, 20, 20), ctx)
    L.CuDNN_conv2d(gx, gw, whole, 1, 1, 1)
    gx.split_tensor(4); parts.split_tensor(4)
    for i in range(4):
        L.CuDNN_conv2d(gx.sTensor[i], gw, parts.sTensor[i], 1, 1, 1)
    np.testing.assert_array_equal(whole.asnumpy(), parts.asnumpy())


@pytest.mark.parametrize("winograd", ["0", None])
def test_conv_full_size_properties(winograd, rng, monkeypatch):
    """Size-independent checks at a full VGG layer shape (64 x 64 x 224 x 224 -> 64, 236.8 GFLOP), on the
    direct kernels and with the routing the library chooses (the Winograd routine): a delta filter copies
    one input channel (exactly on the direct kernels; to a few 1e-7 of the largest value through the
    transforms), and the adjoint identity <conv(x,w),dy> = <x,bwd_data(w,dy)> = <w,bwd_filter(x,dy)> holds."""
    from tsplit_amd import gpu_links as L, ndarray
    if winograd is None:
        monkeypatch.delenv("TSPLIT_CONV_WINOGRAD", raising=False)
        assert L.conv_takes_winograd(64, 64, 64, 224, 224)
    else:
        monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", winograd)
    ctx = ndarray.gpu(0)
    shape = (64, 64, 224, 224)
    # build inputs on the host in float32 without large temporaries
    x = rng.standard_normal(size=shape).astype(np.float32)
    gx = ndarray.array(x, ctx)
    w = np.zeros((64, 64, 3, 3), np.float32)
    perm = rng.permutation(64)
    w[np.arange(64), perm, 1, 1] = 1.0            # output channel o = input channel perm[o]
    y = ndarray.empty(shape, ctx)
    L.CuDNN_conv2d(gx, ndarray.array(w, ctx), y, 1, 1, 1)
    got = y.asnumpy()
    if winograd == "0":
        assert np.array_equal(got, x[:, perm])
    else:
        assert_close(got, x[:, perm], 2e-6, "delta filter through the Winograd transforms")
    del got
    w2 = (rng.standard_normal(size=(64, 64, 3, 3)) / 24.0).astype(np.float32)
    gw2 = ndarray.array(w2, ctx)
    L.CuDNN_conv2d(gx, gw2, y, 1, 1, 1)
    yv = y.asnumpy()
    dy = rng.standard_normal(size=shape).astype(np.float32)
    gdy = ndarray.array(dy, ctx)
    lhs = float(np.vdot(yv.astype(np.float64, copy=False).ravel(), dy.ravel())) if False else float(
        np.sum(yv.reshape(64, -1).astype(np.float64) * dy.reshape(64, -1)))
    dx, dw = ndarray.empty(shape, ctx), ndarray.empty(w2.shape, ctx)
    L.CuDNN_conv2d_gradient_of_data(gw2, gdy, dx, 1, 1, 1)
    L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, 1, 1, 1)
    r1 = float(np.sum(dx.asnumpy().reshape(64, -1).astype(np.float64) * x.reshape(64, -1)))
    r2 = float(np.sum(dw.asnumpy().astype(np.float64) * w2))
    assert abs(r1 - lhs) <= 1e-4 * abs(lhs) and abs(r2 - lhs) <= 1e-4 * abs(lhs), (lhs, r1, r2)


def test_conv_shape_errors():
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    x, w = ndarray.empty((1, 3, 8, 8), ctx), ndarray.empty((4, 3, 3, 3), ctx)
    with pytest.raises(RuntimeError):
        L.CuDNN_conv2d(x, w, ndarray.empty((1, 4, 7, 8), ctx), 1, 1, 1)      # wrong output size
    with pytest.raises(RuntimeError):
        L.CuDNN_conv2d(x, ndarray.empty((4, 2, 3, 3), ctx), ndarray.empty((1, 4, 8, 8), ctx), 1, 1, 1)
