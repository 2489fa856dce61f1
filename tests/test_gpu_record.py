"""Recorded steps: a training step issued once into a HIP graph and replayed with one host call
gives, bit for bit, what issuing the same calls again gives.  (No counterpart in the reference,
whose steps are always issued call by call, python/athena/gpu_ops/executor.py:94-158.)  Every
replay is checked, with eager work and synchronisations between replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _data(shape, classes, seed):
    rng = np.random.RandomState(seed)
    x = rng.standard_normal(shape).astype(np.float32)
    y = np.eye(classes, dtype=np.float32)[rng.randint(0, classes, shape[0])]
    return x, y


def _params_of(t):
    t.sync()
    return {k: v.asnumpy().copy() for k, v in t.params.items()}


def _run_pair(spec, shape, classes, optimizer, steps, fuse=False, between=None):
    """-> (per-step losses and final parameters) of an eager trainer and of a trainer that runs
    its first step eagerly and replays a recording for the others."""
    from tsplit_amd import ndarray, trainer
    x, y = _data(shape, classes, 5)
    out = []
    for recorded in (False, True):
        params = trainer.init_params(spec, seed=11)
        t = trainer.Trainer(spec, params, shape, classes, optimizer=optimizer, fuse_bn_relu=fuse)
        gx, gy = ndarray.array(x, t.ctx), ndarray.array(y, t.ctx)
        losses = []
        t.step(gx, gy)
        losses.append(t.loss_value())
        graph = t.record_step(gx, gy) if recorded else None
        if recorded:
            # recording runs nothing: the loss is still the first step's
            assert t.loss_value() == losses[0]
        for i in range(1, steps):
            if recorded:
                graph.launch(t.stream)
            else:
                t.step(gx, gy)
            losses.append(t.loss_value())              # synchronises between replays
            if between is not None:
                between(t)
        out.append((losses, _params_of(t)))
        del graph, t
    return out


def _assert_same(pair):
    (l0, p0), (l1, p1) = pair
    assert l0 == l1, (l0, l1)
    assert l0[-1] < l0[0]
    for k in p0:
        np.testing.assert_array_equal(p0[k], p1[k], err_msg=k)


def test_mlp_replays_equal_eager_steps():
    from tsplit_amd import trainer
    _assert_same(_run_pair(trainer.mlp_spec(), (128, 784), 10, ("sgd", 0.1), 6))


def test_conv_net_replays_equal_eager_steps_with_eager_work_between():
    """Conv (with tiles cut into pieces and assembled from scratch memory), BatchNorm, Relu, pooling,
    momentum; between replays other kernels run eagerly on the same stream and use the same scratch."""
    from tsplit_amd import gpu_links as L, ndarray
    spec = [("conv", "c1", 3, 16, 3, 1, 1), ("bn", "c1_bn", 16), ("relu",), ("maxpool", 2, 0, 2),
            ("conv", "c2", 16, 32, 3, 1, 1), ("bn", "c2_bn", 32), ("relu",), ("maxpool", 2, 0, 2), ("flatten",),
            ("fc", "f1", 32 * 8 * 8, 10)]
    rng = np.random.RandomState(2)
    xs = rng.standard_normal((4, 16, 20, 20)).astype(np.float32)
    ws = (rng.standard_normal((16, 16, 3, 3)) / 12).astype(np.float32)
    keep = {}

    def between(t):
        if "x" not in keep:
            keep["x"], keep["w"] = ndarray.array(xs, t.ctx), ndarray.array(ws, t.ctx)
            keep["y"] = ndarray.empty((4, 16, 20, 20), t.ctx)
        L.CuDNN_conv2d(keep["x"], keep["w"], keep["y"], 1, 1, 1, t.stream)
        L.relu(keep["y"], keep["y"], t.stream)
        t.sync()

    for fuse in (False, True):
        keep.clear()
        _assert_same(_run_pair(spec, (8, 3, 32, 32), 10, ("momentum", 0.005, 0.9), 5, fuse=fuse, between=between))


def test_replay_reads_the_inputs_of_the_moment():
    """The graph holds addresses, not values: new data copied into the recorded input arrays is what
    the next replay trains on."""
    from tsplit_amd import ndarray, trainer
    spec = trainer.mlp_spec((20, 16, 4))
    xa, ya = _data((8, 20), 4, 1)
    xb, yb = _data((8, 20), 4, 2)
    results = []
    for recorded in (False, True):
        t = trainer.Trainer(spec, trainer.init_params(spec, seed=3), (8, 20), 4, optimizer=("sgd", 0.1))
        gx, gy = ndarray.array(xa, t.ctx), ndarray.array(ya, t.ctx)
        t.step(gx, gy)
        graph = t.record_step(gx, gy) if recorded else None
        t.sync()
        gx[:] = xb
        gy[:] = yb
        if recorded:
            graph.launch(t.stream)
        else:
            t.step(gx, gy)
        results.append((t.loss_value(), _params_of(t)))
    assert results[0][0] == results[1][0]
    for k in results[0][1]:
        np.testing.assert_array_equal(results[0][1][k], results[1][1][k])


def test_tape_step_recorded_keeps_its_temporaries():
    """The define-by-run harness allocates every intermediate while the step is issued; arrays born
    during the recording stay allocated for the graph even after the tape is gone, so later
    allocations cannot land in memory the replays write."""
    import gc
    from tsplit_amd import graph, ndarray, stream, workloads
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState(4)
    x = rng.uniform(0, 1, size=(16, 28 * 28)).astype(np.float32)
    y = np.eye(10, dtype=np.float32)[rng.randint(0, 10, 16)]

    def run(recorded, steps=4):
        st = stream.create_stream_handle(ctx)
        backend = graph.GpuBackend(ctx, st)
        store = workloads.ParamStore(9)
        state = {}

        def one_step():
            t = graph.Tape(backend)
            if "binder" not in state:
                state["binder"] = workloads.Binder(t, store)
                state["inputs"] = {"x": state["binder"].input(x), "y": state["binder"].input(y)}
            else:
                b = state["binder"]
                b.t, b._n = t, 0
                for v in b.vars.values():
                    v.grad = None
            loss, _ = workloads.lstm(t, state["binder"], state["inputs"]["x"], state["inputs"]["y"])
            t.backward(loss)
            state["binder"].sgd_step(0.05)
            return loss

        loss = one_step()
        backend.sync()
        losses = [float(loss.value.asnumpy()[0])]
        if recorded:
            with stream.recording(st) as rec:
                loss = one_step()
            loss_arr = loss.value
            del loss
            gc.collect()
            # fill the pool's free memory with other arrays: none may alias the recorded step's
            junk = [ndarray.array(np.full((1 << 16,), 7.0, np.float32), ctx) for _ in range(32)]
            for _ in range(steps - 1):
                rec.graph.launch(st)
                backend.sync()
                losses.append(float(loss_arr.asnumpy()[0]))
            del junk
        else:
            for _ in range(steps - 1):
                loss = one_step()
                backend.sync()
                losses.append(float(loss.value.asnumpy()[0]))
        state["binder"].pull()
        return losses, {k: v.copy() for k, v in store.values.items()}

    (l0, p0), (l1, p1) = run(False), run(True)
    assert l0 == l1 and l0[-1] < l0[0], (l0, l1)
    for k in p0:
        np.testing.assert_array_equal(p0[k], p1[k], err_msg=k)


def test_first_use_set_up_is_refused_while_recording():
    """A call that would have to grow scratch memory while a step is being recorded fails instead of
    allocating behind the graph's back; the stream works normally afterwards."""
    from tsplit_amd import gpu_links as L, ndarray, stream
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    rng = np.random.RandomState(0)

    def ce_arrays(rows):
        logits = ndarray.array(rng.standard_normal((rows, 4)).astype(np.float32), ctx)
        labels = ndarray.array(np.eye(4, dtype=np.float32)[rng.randint(0, 4, rows)], ctx)
        return logits, labels, ndarray.empty((1,), ctx)

    # the cross-entropy keeps one partial loss per row in per-stream scratch (granules of 1 MiB):
    # 8 rows first, then 300 000 rows, which need more than the first call reserved
    small, large = ce_arrays(8), ce_arrays(300000)
    L.softmax_cross_entropy(small[0], small[1], small[2], st)
    st.sync()
    with pytest.raises(RuntimeError):
        with stream.recording(st):
            L.softmax_cross_entropy(large[0], large[1], large[2], st)
    # eager again: allowed to grow now, and correct
    L.softmax_cross_entropy(large[0], large[1], large[2], st)
    st.sync()
    z = large[0].asnumpy().astype(np.float64)
    lse = np.log(np.exp(z - z.max(1, keepdims=True)).sum(1)) + z.max(1)
    ref = float(np.mean(lse - (z * large[1].asnumpy()).sum(1)))
    assert abs(float(large[2].asnumpy()[0]) - ref) <= 1e-4 * abs(ref)


def test_scratch_growing_after_a_recording_leaves_the_graph_its_buffer():
    """A recorded step holds the address of the scratch buffer it was recorded with.  When a later
    eager call on the same stream needs more scratch than that, the library takes a new buffer for
    the stream and keeps the recorded one allocated until the graph is destroyed, so replays after
    the growth still compute the same values (softmax cross-entropy keeps one partial loss per row
    in per-stream scratch, in granules of 1 MiB)."""
    from tsplit_amd import gpu_links as L, ndarray, stream
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    rng = np.random.RandomState(4)

    def ce_arrays(rows):
        logits = ndarray.array(rng.standard_normal((rows, 4)).astype(np.float32), ctx)
        labels = ndarray.array(np.eye(4, dtype=np.float32)[rng.randint(0, 4, rows)], ctx)
        return logits, labels, ndarray.empty((1,), ctx)

    small, large = ce_arrays(1000), ce_arrays(600000)
    L.softmax_cross_entropy(small[0], small[1], small[2], st)          # first use: scratch of 1 MiB
    st.sync()
    want = small[2].asnumpy().copy()
    with stream.recording(st) as rec:
        L.softmax_cross_entropy(small[0], small[1], small[2], st)
    for _ in range(3):
        L.array_set(small[2], -1.0, st)
        rec.graph.launch(st)
        st.sync()
        np.testing.assert_array_equal(small[2].asnumpy(), want)
        # eager work on the same stream that needs more than the recorded buffer holds (2.4 MB of
        # row losses), then other allocations that could land where a freed buffer was
        L.softmax_cross_entropy(large[0], large[1], large[2], st)
        st.sync()
        filler = [ndarray.array(np.full((1 << 18,), 7.0, np.float32), ctx) for _ in range(4)]
        del filler
    z = large[0].asnumpy().astype(np.float64)
    lse = np.log(np.exp(z - z.max(1, keepdims=True)).sum(1)) + z.max(1)
    ref = float(np.mean(lse - (z * large[1].asnumpy()).sum(1)))
    assert abs(float(large[2].asnumpy()[0]) - ref) <= 1e-4 * abs(ref)
    del rec
