"""The entry point that allocates nothing: TSplit_SoftmaxCrossEntropyNoAlloc keeps its per-row losses in
a fixed array inside the library instead of the library's grow-on-demand scratch memory.  It runs the
same kernels as DLGpuSoftmaxCrossEntropy, so its loss must equal that call's bit for bit: on two calls in
a row, the second with a smaller input (the array keeps the first call's contents), for short rows (one
wavefront per row) and long ones (one block per row), from the NULL stream and from a created one, and it
must refuse more rows than the array holds."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MAX_ROWS = 1 << 18


def _no_alloc(logits, labels, out, stream=None):
    from tsplit_amd._base import _LIB
    return _LIB.TSplit_SoftmaxCrossEntropyNoAlloc(logits.handle, labels.handle, out.handle, stream.handle if stream else None)


def _case(rng, rows, cols, ctx):
    from tsplit_amd import ndarray
    z = (3.0 * rng.standard_normal((rows, cols))).astype(np.float32)
    lab = np.zeros((rows, cols), np.float32)
    lab[np.arange(rows), rng.randint(0, cols, rows)] = 1.0
    return z, lab, ndarray.array(z, ctx), ndarray.array(lab, ctx)


@pytest.mark.parametrize("shapes", [((4096, 1000), (37, 1000)), ((300, 4096), (5, 4096)), ((MAX_ROWS, 8), (1, 8))])
def test_no_alloc_loss_equals_the_allocating_call_twice_in_a_row(shapes):
    from oracle import ops as O
    from tsplit_amd import gpu_links as L, ndarray, stream
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    rng = np.random.RandomState(17)
    for use_stream in (None, st):
        for rows, cols in shapes:                    # the second call is the smaller one
            z, lab, gz, glab = _case(rng, rows, cols, ctx)
            want, got = ndarray.empty((1,), ctx), ndarray.empty((1,), ctx)
            L.array_set(got, -7.0, use_stream)
            L.softmax_cross_entropy(gz, glab, want, use_stream)
            assert _no_alloc(gz, glab, got, use_stream) == 0
            if use_stream:
                use_stream.sync()
            a, b = want.asnumpy(), got.asnumpy()
            assert a.tobytes() == b.tobytes(), (rows, cols, a, b)
            ref = O.softmax_ce(z, lab)
            assert abs(float(b[0]) - float(ref[0])) <= 1e-4 * abs(float(ref[0]))


def test_no_alloc_refuses_more_rows_than_its_array_holds(capfd):
    from tsplit_amd import ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState(3)
    _, _, gz, glab = _case(rng, MAX_ROWS + 1, 4, ctx)
    out = ndarray.empty((1,), ctx)
    assert _no_alloc(gz, glab, out) == -1
    assert "fixed scratch array" in capfd.readouterr().err


def test_no_alloc_call_allocates_no_device_memory():
    """What the entry point is for: after the library's init call and one warm-up call, a call changes
    neither the device pool's accounting nor the device's free memory (hipMemGetInfo, asked through the
    HIP runtime the library itself is linked against)."""
    from tsplit_amd import gpu_links as L, gpu_memory_manager as M, ndarray, stream
    from tsplit_amd._base import _LIB
    hip = ctypes.CDLL("libamdhip64.so")
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    _LIB.cudnn_init(0, None)                      # void in the reference ABI; looks the array up on device 0

    def device_free():
        free, total = ctypes.c_size_t(), ctypes.c_size_t()
        assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
        return free.value

    rng = np.random.RandomState(5)
    cases = [_case(rng, 2048, 1000, ctx), _case(rng, 64, 4096, ctx)]
    out = ndarray.empty((1,), ctx)
    for _, _, gz, glab in cases:                       # warm-up: code objects loaded, kernels resolved
        assert _no_alloc(gz, glab, out, st) == 0
    st.sync()
    pool_before, free_before = M.pool_state(), device_free()
    for _ in range(3):
        for _, _, gz, glab in cases:
            assert _no_alloc(gz, glab, out, st) == 0
            assert _no_alloc(gz, glab, out, None) == 0
    st.sync()
    assert M.pool_state() == pool_before
    assert device_free() == free_before
