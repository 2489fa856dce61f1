"""Run-to-run determinism: nothing in the operator library depends on scheduling (cut tiles are
assembled in block order, split-K slices folded in a fixed order, no float atomics on the training
path), so two runs of the same training steps from the same state give the same bits - losses and
every parameter - also when another stream keeps the GPU busy with unrelated convolutions."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

# shapes chosen so that the convolutions cut tiles between blocks, split K in the filter gradient,
# use both tile families, a strided layer and padded image tails
SPEC = [("conv", "c1", 3, 64, 3, 1, 1), ("bn", "c1_bn", 64), ("relu",),
        ("conv", "c2", 64, 64, 3, 1, 1), ("bn", "c2_bn", 64), ("relu",), ("maxpool", 2, 0, 2),
        ("conv", "c3", 64, 192, 3, 1, 1), ("bn", "c3_bn", 192), ("relu",),
        ("conv", "c4", 192, 128, 3, 1, 2), ("bn", "c4_bn", 128), ("relu",),
        ("conv", "c5", 128, 256, 1, 0, 1), ("bn", "c5_bn", 256), ("relu",), ("maxpool", 2, 0, 2),
        ("flatten",), ("fc", "f1", 256 * 7 * 7, 100), ("fc", "f2", 100, 10)]


def _train(steps, busy):
    from tsplit_amd import gpu_links as L, ndarray, stream, trainer
    rng = np.random.RandomState(17)
    x = rng.standard_normal((24, 3, 54, 54)).astype(np.float32)
    y = np.eye(10, dtype=np.float32)[rng.randint(0, 10, 24)]
    t = trainer.Trainer(SPEC, trainer.init_params(SPEC, seed=5, scheme="he"), x.shape, 10,
                        optimizer=("momentum", 1e-4, 0.9), split={3: 2})
    gx, gy = ndarray.array(x, t.ctx), ndarray.array(y, t.ctx)
    other = None
    if busy:
        other = stream.create_stream_handle(t.ctx)
        bx = ndarray.array(rng.standard_normal((8, 64, 40, 40)).astype(np.float32), t.ctx)
        bw = ndarray.array((rng.standard_normal((96, 64, 3, 3)) / 24).astype(np.float32), t.ctx)
        by = ndarray.empty((8, 96, 40, 40), t.ctx)
    losses = []
    for _ in range(steps):
        if busy:
            for _ in range(6):
                L.CuDNN_conv2d(bx, bw, by, 1, 1, 1, other)
        t.step(gx, gy)
        losses.append(t.loss_value())
    if busy:
        other.sync()
    t.sync()
    return losses, {k: v.asnumpy().copy() for k, v in t.params.items()}


def test_training_steps_repeat_bit_for_bit():
    first = _train(3, busy=False)
    again = _train(3, busy=False)
    crowded = _train(3, busy=True)
    assert np.isfinite(first[0]).all() and len(set(first[0])) == 3      # the steps do change the net
    for other in (again, crowded):
        assert other[0] == first[0]
        for k in first[1]:
            np.testing.assert_array_equal(other[1][k], first[1][k], err_msg=k)
