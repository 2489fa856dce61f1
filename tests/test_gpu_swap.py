"""The swap path the memory-policy executors rely on (python/athena/ndarray.py:221-243,
gpu_ops/vdnnExecutor.py:202-330): pinned host arrays from the host pool, DLArrayCopyFromTo on a
copy stream, events to order the copy against compute.  Copies are bit-exact."""
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    from tsplit_amd import gpu_links, ndarray, stream
    ctx = ndarray.gpu(0)

    class NS:
        pass
    ns = NS()
    ns.nd, ns.links, ns.ctx = ndarray, gpu_links, ctx
    ns.compute = stream.create_stream_handle(ctx)
    ns.copy = stream.create_stream_handle(ctx)
    ns.event = lambda: stream.create_event_handle(ctx)
    return ns


def test_host_arrays_come_from_a_pinned_pool(env):
    nd = env.nd
    a = nd.empty((1 << 20,), nd.cpu(0))
    p1 = a.data_ptr
    del a
    b = nd.empty((1 << 20,), nd.cpu(0))
    assert b.data_ptr == p1                     # the freed chunk is handed out again
    c = nd.empty((1 << 18,), nd.cpu(0))
    assert c.data_ptr != b.data_ptr
    t0 = time.perf_counter()
    keep = [nd.empty((1 << 16,), nd.cpu(0)) for _ in range(200)]
    dt = (time.perf_counter() - t0) / 200
    assert dt < 100e-6, "host allocation takes %.0f us: not pooled" % (dt * 1e6)
    assert len({k.data_ptr for k in keep}) == 200


def test_async_swap_out_and_in_round_trip(env, rng):
    nd = env.nd
    x = rng.normal(size=(8, 64, 56, 56)).astype(np.float32)
    g = nd.array(x, env.ctx)
    host = nd.empty(x.shape, nd.cpu(0))
    out_done, in_done = env.event(), env.event()
    host.async_d2h(g, env.copy, out_done)       # swap out
    out_done.sync()
    assert out_done.query()
    np.testing.assert_array_equal(host.asnumpy(), x)
    env.links.array_set(g, 0.0, env.compute)     # the device copy is gone
    env.compute.sync()
    g.async_h2d(host, env.copy, in_done)        # swap in
    in_done.sync()
    np.testing.assert_array_equal(g.asnumpy(), x)


def test_copies_overlap_compute_without_disturbing_it(env, rng):
    """A convolution runs on the compute stream while activations of another layer are swapped
    out and back in on the copy stream; both streams produce exact results."""
    from oracle import ops as O
    nd, L = env.nd, env.links
    x = rng.normal(size=(8, 32, 28, 28)).astype(np.float32)
    w = (rng.normal(size=(32, 32, 3, 3)) / 17).astype(np.float32)
    gx, gw, gy = nd.array(x, env.ctx), nd.array(w, env.ctx), nd.empty((8, 32, 28, 28), env.ctx)
    act = rng.normal(size=(64, 64, 56, 56)).astype(np.float32)      # 51 MB
    gact = nd.array(act, env.ctx)
    host = nd.empty(act.shape, nd.cpu(0))
    back = nd.empty(act.shape, env.ctx)
    ev_out, ev_in = env.event(), env.event()
    for _ in range(20):
        L.CuDNN_conv2d(gx, gw, gy, 1, 1, 1, env.compute)
    host.async_d2h(gact, env.copy, ev_out)
    back.async_h2d(host, env.copy, ev_in)       # same stream: ordered after the swap-out
    for _ in range(20):
        L.CuDNN_conv2d(gx, gw, gy, 1, 1, 1, env.compute)
    ev_in.sync()
    env.compute.sync()
    np.testing.assert_array_equal(back.asnumpy(), act)
    ref = O.conv2d(x, w, 1, 1, 1)
    assert np.max(np.abs(gy.asnumpy() - ref)) <= 2e-3 * np.max(np.abs(ref))
