"""SGDOptimizerUpdate / MomentumOptimizerUpdate put their arrays on a list that runs as one launch when anything else is
asked of the library (csrc/common.h).  Whatever the caller does next must see every update done, in order, with the
bits of one launch per parameter."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ts():
    import types
    from tsplit_amd import gpu_links, ndarray, stream
    ns = types.SimpleNamespace()
    ns.L, ns.nd = gpu_links, ndarray
    ns.ctx = ndarray.gpu(0)
    ns.stream = stream.create_stream_handle(ns.ctx)
    ns.other = stream.create_stream_handle(ns.ctx)
    ns.arr = lambda a: ndarray.array(np.asarray(a, np.float32), ns.ctx)
    return ns


SIZES = [1, 3, 64, 257, 4096, 100003, 1 << 20, 7, 512, 512, 25088 * 64]


def _params(rng):
    return [(rng.normal(size=n).astype(np.float32), rng.normal(size=n).astype(np.float32), rng.normal(size=n).astype(np.float32))
            for n in SIZES]


@pytest.mark.parametrize("rule", ["sgd", "momentum", "nesterov"])
def test_a_list_of_updates_has_the_bits_of_one_launch_per_parameter(ts, rule):
    """The same updates issued back to back (one list, one launch) and with a stream synchronisation after each
    (every list has one entry and runs as the single-array launch)."""
    rng = np.random.RandomState(3)
    host = _params(rng)
    results = []
    for eager in (False, True):
        dev = [(ts.arr(p), ts.arr(g), ts.arr(v)) for p, g, v in host]
        for _ in range(2):                       # two steps: the second list is the one the library has kept
            for p, g, v in dev:
                if rule == "sgd":
                    ts.L.sgd_update(p, g, 0.05, ts.stream)
                else:
                    ts.L.momentum_update(p, g, v, 0.05, 0.9, rule == "nesterov", ts.stream)
                if eager:
                    ts.stream.sync()
            ts.stream.sync()
        results.append([(p.asnumpy(), v.asnumpy()) for p, g, v in dev])
    for (p0, v0), (p1, v1), (hp, hg, hv) in zip(results[0], results[1], host):
        np.testing.assert_array_equal(p0, p1)
        np.testing.assert_array_equal(v0, v1)
        assert not np.array_equal(p0, hp)
    # and against the arithmetic itself
    p, g, v = (a.astype(np.float64) for a in host[4])
    for _ in range(2):
        if rule == "sgd":
            p = p - 0.05 * g
        elif rule == "nesterov":                 # the reference's form (src/ops/Optimizers.cu:80-85)
            v = 0.9 * (v - 0.05 * g)
            p = p + v - 0.05 * g
        else:
            v = 0.9 * v - 0.05 * g
            p = p + v
    assert np.max(np.abs(results[0][4][0] - p)) <= 1e-5 * np.max(np.abs(p))


def test_updates_of_one_parameter_keep_their_order(ts):
    """The same parameter twice in a row, with the same and with another rate, and a gradient that is itself updated
    in between: a list never holds two entries that touch the same memory."""
    rng = np.random.RandomState(4)
    p0, g0, h0 = (rng.normal(size=1000).astype(np.float32) for _ in range(3))
    p, g, h = ts.arr(p0), ts.arr(g0), ts.arr(h0)
    ts.L.sgd_update(p, g, 0.1, ts.stream)
    ts.L.sgd_update(p, g, 0.1, ts.stream)        # same arrays, same rate
    ts.L.sgd_update(p, g, 0.3, ts.stream)        # another rate
    ts.L.sgd_update(g, h, 0.5, ts.stream)        # writes what the entries above read
    ts.L.sgd_update(p, g, 0.1, ts.stream)        # reads what the entry above writes
    ref_p = ((p0 - np.float32(0.1) * g0) - np.float32(0.1) * g0) - np.float32(0.3) * g0
    ref_g = g0 - np.float32(0.5) * h0
    ref_p = ref_p - np.float32(0.1) * ref_g
    assert np.max(np.abs(p.asnumpy() - ref_p)) <= 2e-6 * np.max(np.abs(ref_p))
    assert np.max(np.abs(g.asnumpy() - ref_g)) <= 2e-6 * np.max(np.abs(ref_g))
    # a micro-tensor view of a parameter and the parameter itself
    big = ts.arr(rng.normal(size=(8, 100)).astype(np.float32))
    big0 = big.asnumpy()
    gb = ts.arr(np.ones((8, 100), np.float32))
    big.split_tensor(4)
    gb.split_tensor(4)
    ts.L.sgd_update(big.sTensor[1], gb.sTensor[1], 1.0, ts.stream)
    ts.L.sgd_update(big, gb, 1.0, ts.stream)
    want = big0 - 1.0
    want[2:4] -= 1.0
    np.testing.assert_allclose(big.asnumpy(), want, rtol=0, atol=1e-6)


def test_an_array_may_be_freed_or_overwritten_right_after_its_update(ts):
    rng = np.random.RandomState(5)
    p0 = rng.normal(size=5000).astype(np.float32)
    g0 = rng.normal(size=5000).astype(np.float32)
    p = ts.arr(p0)
    g = ts.arr(g0)
    ts.L.sgd_update(p, g, 0.25, ts.stream)
    del g                                        # DLArrayFree: the list runs first
    junk = [ts.arr(np.full(5000, 1e9, np.float32)) for _ in range(4)]      # may take the freed memory
    np.testing.assert_array_equal(p.asnumpy(), p0 - np.float32(0.25) * g0)
    # overwriting the gradient through the library right after the call
    g2 = ts.arr(g0)
    ts.L.sgd_update(p, g2, 0.25, ts.stream)
    ts.L.array_set(g2, 0.0, ts.stream)
    ts.L.sgd_update(p, g2, 0.25, ts.stream)
    want = (p0 - np.float32(0.25) * g0) - np.float32(0.25) * g0
    np.testing.assert_array_equal(p.asnumpy(), want)
    del junk


def test_another_stream_sees_the_update_behind_an_event(ts):
    from tsplit_amd import stream as S
    rng = np.random.RandomState(6)
    p0, g0 = rng.normal(size=1 << 16).astype(np.float32), rng.normal(size=1 << 16).astype(np.float32)
    p, g = ts.arr(p0), ts.arr(g0)
    copy = ts.nd.empty((1 << 16,), ts.ctx)
    ts.L.sgd_update(p, g, 0.5, ts.stream)
    ev = S.create_event_handle(ts.ctx)
    ev.record(ts.stream)                         # the list runs in front of the event
    ev.sync()
    p.copyto(copy, ts.other)
    ts.other.sync()
    np.testing.assert_array_equal(copy.asnumpy(), p0 - np.float32(0.5) * g0)
    # the default stream (no handle)
    ts.L.sgd_update(p, g, 0.5, None)
    np.testing.assert_array_equal(p.asnumpy(), (p0 - np.float32(0.5) * g0) - np.float32(0.5) * g0)


def test_lists_that_change_from_call_to_call(ts):
    """Two sets of parameters updated in turn, and lists of a different length every time: the table of arrays the
    one launch reads is uploaded again each time, through staging buffers that take turns."""
    rng = np.random.RandomState(7)
    sizes = [4, 1000, 4096, 33000, 64, 12, 70000, 256]
    host = [(rng.normal(size=n).astype(np.float32), rng.normal(size=n).astype(np.float32)) for n in sizes]
    dev = [(ts.arr(p), ts.arr(g)) for p, g in host]
    want = [p.copy() for p, _ in host]
    lr = np.float32(0.125)
    for round_ in range(12):
        chosen = [i for i in range(len(sizes)) if (i + round_) % 2 == 0][:2 + round_ % 3]
        for i in chosen:
            ts.L.sgd_update(dev[i][0], dev[i][1], float(lr), ts.stream)
            want[i] = want[i] - lr * host[i][1]
        ts.L.array_set(ts.arr(np.zeros(4, np.float32)), 1.0, ts.stream)      # any other call: the list runs
    for (p, _), w in zip(dev, want):
        np.testing.assert_array_equal(p.asnumpy(), w)
