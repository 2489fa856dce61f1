"""CuDNN_DLGpuBatch_Normalization right behind the convolution that produced its input takes its batch
statistics from the sums that convolution's epilogue left (one read of the tensor instead of two).  Held
here: the result against the oracle and against the call without the shortcut (1e-4 / 1e-6); that the
shortcut is really taken in the situations of a training step (one convolution, the convolutions of
consecutive batch micro-tensors, the fused BatchNorm + Relu call); and that sums are NEVER used once the
tensor may have changed - overwritten through a device copy with or without a stream, through another
operator writing in place, through a host upload, by a second convolution into the same array - or when
the BatchNorm runs on another stream, on a part or a superset of the range, or after any other operator."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close, assert_close_entries

pytestmark = pytest.mark.gpu
EPS = 0.01


@pytest.fixture(scope="module")
def ts():
    from tsplit_amd import gpu_links, ndarray, stream
    ctx = ndarray.gpu(0)

    class NS:
        pass
    ns = NS()
    ns.L, ns.nd, ns.ctx = gpu_links, ndarray, ctx
    ns.stream = stream.create_stream_handle(ctx)
    ns.other = stream.create_stream_handle(ctx)
    ns.arr = lambda a: ndarray.array(np.asarray(a, np.float32), ctx)
    ns.empty = lambda shape: ndarray.empty(shape, ctx)
    return ns


def _served(ts):
    return ts.L.batch_norm_look_behind()[0]


def _layer(rng, n=8, c=64, o=64, hw=128):
    """A layer the Winograd routine takes (its epilogue sums per channel) and whose output, 8 x 64 x 128 x 128 = 32 MiB,
    is large enough for a note (smaller outputs leave none: the pass a note saves costs no more than the fold launch)."""
    x = rng.normal(size=(n, c, hw, hw)).astype(np.float32)
    w = (rng.normal(size=(o, c, 3, 3)) / np.sqrt(9 * c)).astype(np.float32)
    g = rng.normal(size=(1, o, 1, 1)).astype(np.float32)
    b = rng.normal(size=(1, o, 1, 1)).astype(np.float32)
    return x, w, g, b


def _bn(ts, y, g, b, stream=None):
    out = ts.empty(y.shape)
    ts.L.CuDNN_Batch_Normalization(y, g, b, out, None, None, 0.99, EPS, stream or ts.stream)
    return out.asnumpy()


def test_batchnorm_behind_a_convolution_uses_its_sums_and_matches_the_oracle(ts, rng):
    x, w, g, b = _layer(rng)
    gx, gw, gg, gb = ts.arr(x), ts.arr(w), ts.arr(g), ts.arr(b)
    y = ts.empty((8, 64, 128, 128))
    assert ts.L.conv_takes_winograd(8, 64, 64, 128, 128)
    before = _served(ts)
    ts.L.CuDNN_conv2d(gx, gw, y, 1, 1, 1, ts.stream)
    assert ts.L.batch_norm_look_behind()[1]                 # a note is pending
    got = _bn(ts, y, gg, gb)
    assert _served(ts) == before + 1 and not ts.L.batch_norm_look_behind()[1]
    conv = y.asnumpy()
    assert_close_entries(got, O.batchnorm_forward(conv, g, b, EPS)[0], 1e-4, "BatchNorm from the convolution's sums")
    again = _bn(ts, y, gg, gb)                                # the note is gone: the ordinary two passes
    assert _served(ts) == before + 1
    assert_close(got, again, 1e-6, "with and without the shortcut")
    # the direct (tap-major) kernels leave sums too: 1x1 filter, 128 -> 128
    x1 = rng.normal(size=(8, 128, 96, 96)).astype(np.float32)
    w1 = (rng.normal(size=(128, 128, 1, 1)) / np.sqrt(128)).astype(np.float32)
    g1, b1 = rng.normal(size=(1, 128, 1, 1)).astype(np.float32), rng.normal(size=(1, 128, 1, 1)).astype(np.float32)
    y1, gx1, gw1, gg1, gb1 = ts.empty((8, 128, 96, 96)), ts.arr(x1), ts.arr(w1), ts.arr(g1), ts.arr(b1)
    ts.L.CuDNN_conv2d(gx1, gw1, y1, 0, 0, 1, ts.stream)       # (an upload between the two calls would end the note)
    got1 = _bn(ts, y1, gg1, gb1)
    assert _served(ts) == before + 2
    assert_close_entries(got1, O.batchnorm_forward(y1.asnumpy(), g1, b1, EPS)[0], 1e-4, "behind a direct kernel")


def test_micro_tensor_convolutions_add_up_and_the_fused_call_takes_them_too(ts, rng):
    # 32 images in four micro-tensors of 8: every piece is large enough for a note
    x, w, g, b = _layer(rng, n=32)
    gx, gw, gg, gb = ts.arr(x), ts.arr(w), ts.arr(g), ts.arr(b)
    y = ts.empty((32, 64, 128, 128))
    gx.split_tensor(4)
    y.split_tensor(4)
    before = _served(ts)
    for i in range(4):
        ts.L.CuDNN_conv2d(gx.sTensor[i], gw, y.sTensor[i], 1, 1, 1, ts.stream)
    got = _bn(ts, y, gg, gb)
    assert _served(ts) == before + 1
    conv = y.asnumpy()
    ref, mean, var = O.batchnorm_forward(conv, g, b, EPS)
    assert_close_entries(got, ref, 1e-4, "BatchNorm over four micro-tensors' sums")
    # pieces out of order: no shortcut, same result
    for i in (1, 0, 2, 3):
        ts.L.CuDNN_conv2d(gx.sTensor[i], gw, y.sTensor[i], 1, 1, 1, ts.stream)
    assert_close(_bn(ts, y, gg, gb), got, 1e-6, "pieces out of order")
    assert _served(ts) == before + 1
    # a BatchNorm over ONE micro-tensor sees that micro-tensor's sums only, and all notes end with it
    for i in range(4):
        ts.L.CuDNN_conv2d(gx.sTensor[i], gw, y.sTensor[i], 1, 1, 1, ts.stream)
    one = _bn(ts, y.sTensor[2], gg, gb)
    assert _served(ts) == before + 2 and not ts.L.batch_norm_look_behind()[1]
    assert_close_entries(one, O.batchnorm_forward(conv[16:24], g, b, EPS)[0], 1e-4, "one micro-tensor")
    # the fused BatchNorm + Relu symbol
    for i in range(4):
        ts.L.CuDNN_conv2d(gx.sTensor[i], gw, y.sTensor[i], 1, 1, 1, ts.stream)
    out, sm, sv = ts.empty(y.shape), ts.empty((1, 64, 1, 1)), ts.empty((1, 64, 1, 1))
    ts.L.batch_norm_relu(y, gg, gb, out, sm, sv, EPS, stream=ts.stream)
    assert _served(ts) == before + 3
    assert_close(out.asnumpy(), np.maximum(ref, 0), 1e-4, "fused BatchNorm + Relu from the sums")
    assert_close(sm.asnumpy().ravel(), mean, 1e-4, "saved mean")
    assert_close(sv.asnumpy().ravel(), 1 / np.sqrt(var + EPS), 1e-4, "saved inverse deviation")


def test_small_outputs_leave_no_note(ts, rng):
    """At most 16 384 values per channel (the BatchNorm reads such a tensor once anyway) or less than 32 MiB in all (the
    saved pass is no longer than the extra launch): the convolution neither sums nor notes."""
    for n, hw in ((4, 56), (8, 56), (4, 128)):
        _no_note(ts, rng, n, hw)


def _no_note(ts, rng, n, hw):
    x, w, g, b = _layer(rng, n=n, hw=hw)
    gx, gw, gg, gb = ts.arr(x), ts.arr(w), ts.arr(g), ts.arr(b)
    y = ts.empty((n, 64, hw, hw))
    before = _served(ts)
    ts.L.CuDNN_conv2d(gx, gw, y, 1, 1, 1, ts.stream)
    assert not ts.L.batch_norm_look_behind()[1]
    got = _bn(ts, y, gg, gb)
    assert _served(ts) == before
    assert_close_entries(got, O.batchnorm_forward(y.asnumpy(), g, b, EPS)[0], 1e-4, "small tensor, no note")


@pytest.mark.parametrize("how", ["device copy on the stream", "device copy without a stream", "host upload", "operator in place",
                                 "second convolution into the array", "another stream", "part of the range", "unrelated operator"])
def test_sums_are_never_used_once_the_tensor_may_have_changed(ts, how, rng):
    x, w, g, b = _layer(rng)
    gx, gw, gg, gb = ts.arr(x), ts.arr(w), ts.arr(g), ts.arr(b)
    y = ts.empty((8, 64, 128, 128))
    other = rng.normal(size=(8, 64, 128, 128)).astype(np.float32) * 3 + 1
    g_other = ts.arr(other)
    before = _served(ts)
    ts.L.CuDNN_conv2d(gx, gw, y, 1, 1, 1, ts.stream)
    assert ts.L.batch_norm_look_behind()[1]
    expect_from = None
    if how == "device copy on the stream":
        g_other.copyto(y, ts.stream)
        expect_from = other
    elif how == "device copy without a stream":
        ts.stream.sync()
        g_other.copyto(y)
        expect_from = other
    elif how == "host upload":
        ts.stream.sync()
        y._sync_copyfrom(other)
        expect_from = other
    elif how == "operator in place":
        ts.L.matrix_elementwise_multiply_by_const(y, -2.0, y, ts.stream)
    elif how == "second convolution into the array":
        # (its own note replaces the first one: the shortcut is taken, with the second convolution's sums)
        w2 = (rng.normal(size=(64, 64, 3, 3)) / 5).astype(np.float32)
        ts.L.CuDNN_conv2d(gx, ts.arr(w2), y, 1, 1, 1, ts.stream)
    elif how == "another stream":
        ts.stream.sync()
        got = _bn(ts, y, gg, gb, ts.other)
        assert _served(ts) == before
        assert_close_entries(got, O.batchnorm_forward(y.asnumpy(), g, b, EPS)[0], 1e-4, how)
        return
    elif how == "part of the range":
        y.split_tensor(2)
        got = _bn(ts, y.sTensor[0], gg, gb)
        assert _served(ts) == before
        assert_close_entries(got, O.batchnorm_forward(y.asnumpy()[:4], g, b, EPS)[0], 1e-4, how)
        return
    elif how == "unrelated operator":
        ts.L.relu(g_other, g_other, ts.stream)
    if how != "second convolution into the array":
        assert not ts.L.batch_norm_look_behind()[1], how          # the note ended with the call in between
    got = _bn(ts, y, gg, gb)
    assert _served(ts) == before + (1 if how == "second convolution into the array" else 0)
    now = y.asnumpy()
    if expect_from is not None:
        np.testing.assert_array_equal(now, expect_from)
    assert_close_entries(got, O.batchnorm_forward(now, g, b, EPS)[0], 1e-4, how)
