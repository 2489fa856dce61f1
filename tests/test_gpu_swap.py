"""The swap path the memory-policy executors rely on (python/athena/ndarray.py:221-243,
gpu_ops/vdnnExecutor.py:202-330): pinned host arrays from the host pool, DLArrayCopyFromTo on a
copy stream, events to order the copy against compute.  Copies are bit-exact."""
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
    # 200 arrays of 256 KiB are carved out of a slab next to one another, not allocated one by one
    keep = [nd.empty((1 << 16,), nd.cpu(0)) for _ in range(200)]
    ptrs = sorted(k.data_ptr for k in keep)
    assert len(set(ptrs)) == 200 and all(p % 256 == 0 for p in ptrs)
    gaps = [b - a for a, b in zip(ptrs, ptrs[1:])]
    assert sum(1 for g in gaps if g == 4 << 16) >= 190, "host arrays are not neighbours in a slab"


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


def test_raw_allocation_rule_runs_the_same_step():
    """MEMORY_MANAGE_RULE 0 (one device malloc / free per tensor, host arrays unpinned) and the
    pooled rule give the same training step bit for bit: the rule only decides where bytes live."""
    import numpy as np
    from tsplit_amd import ndarray, trainer
    spec = [("conv", "c1", 3, 8, 3, 1, 1), ("bn", "c1_bn", 8), ("relu",), ("maxpool", 2, 0, 2), ("flatten",),
            ("fc", "f1", 8 * 8 * 8, 10)]
    rng = np.random.RandomState(3)
    x = rng.standard_normal((4, 3, 16, 16)).astype(np.float32)
    y = np.eye(10, dtype=np.float32)[rng.randint(0, 10, 4)]
    losses = {}
    saved = ndarray.MEMORY_MANAGE_RULE
    try:
        for rule in (1, 0):
            ndarray.MEMORY_MANAGE_RULE = rule
            params = trainer.init_params(spec, seed=7)
            t = trainer.Trainer(spec, params, x.shape, 10, optimizer=("momentum", 0.05, 0.9))
            gx, gy = ndarray.array(x, t.ctx), ndarray.array(y, t.ctx)
            out = []
            for _ in range(3):
                t.step(gx, gy)
                out.append(t.loss_value())
            losses[rule] = out
            host = ndarray.empty((8,), ndarray.cpu(0))          # a host array under the same rule
            host[:] = np.arange(8, dtype=np.float32)
            assert list(host.asnumpy()) == list(range(8))
            del t, gx, gy, host
    finally:
        ndarray.MEMORY_MANAGE_RULE = saved
    assert losses[0] == losses[1] and losses[0][-1] < losses[0][0]
