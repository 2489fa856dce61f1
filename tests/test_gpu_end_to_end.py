"""End-to-end parity: whole training runs through the C ABI track the CPU oracle.
Tolerance from the task statement: loss within 1e-3 relative over 20 steps."""
import numpy as np
import pytest

from oracle import nets, ops as O
from util import assert_close

pytestmark = pytest.mark.gpu


def _onehot(idx, n):
    return np.eye(n, dtype=np.float32)[idx]


def test_mlp_20_steps_tracks_oracle():
    """The reference's CPU-runnable MLP: 784-256-256-10 without bias, batch 128, 20 SGD steps, lr 0.1,
    X ~ U[0,1), labels uniform, weights ~ N(0, 0.1)."""
    from tsplit_amd import ndarray, trainer
    rng = np.random.RandomState(123)
    X = rng.uniform(0, 1, (128, 784)).astype(np.float32)
    Y = _onehot(rng.randint(0, 10, 128), 10)
    spec = trainer.mlp_spec()
    params = {k: rng.normal(0, 0.1, s).astype(np.float32) for k, s in trainer.param_shapes(spec).items()}
    ref_losses, ref_params = nets.train(spec, params, X, Y, steps=20, lr=0.1)
    ctx = ndarray.gpu(0)
    t = trainer.Trainer(spec, params, X.shape, 10, ctx, optimizer=("sgd", 0.1))
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for _ in range(20):
        t.step(gx, gy)
        losses.append(t.loss_value())
    rel = np.max(np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses))
    assert rel <= 1e-3, (rel, losses, ref_losses)
    assert ref_losses[-1] < ref_losses[0]            # it does train
    for k in params:
        assert_close(t.params[k].asnumpy(), ref_params[k], 1e-3, k)


VGG_20_STEP_LR = 5e-7
# Yardstick for quantities that are not stable functions of rounding (end-to-end gradients through
# Relu / pooling decisions, the sum of 20 updates): the distance of the float32 run of the oracle from
# its float64 run is what fp32 arithmetic by itself does to them; the GPU result may sit at most
# YARDSTICK_FACTOR times as far from the float64 run (both measured norm-wise, relative to the float64
# result), plus a floor of the operator tolerance for quantities fp32 arithmetic happens to hit.
# Measured on VGG-16 at 224x224: the float32 oracle sits 0.37 - 0.49 % from the float64 gradients, the
# device 1.0 - 1.24 % (2.3 - 3.1 times as far; the old fixed bar was 25 %).  The factor is above 2 for a
# reason that can be named: the distance comes from Relu / pooling decisions that flip, their number
# grows with the operators' own rounding error, and the Winograd routine's (about 1e-5 of the output,
# inside the 2e-3 operator bar) is ten times a float32 direct sum's, so about sqrt(10) times the
# distance is what the arithmetic predicts.
YARDSTICK_FACTOR = 3.0
YARDSTICK_FLOOR = 2e-3
LAST_STEP_LOSS_BAR = 1e-4     # measured: 2e-6 on the direct kernels, 2e-5 through the Winograd routine


def _small_convnet():
    return [("conv", "c1", 3, 8, 3, 1, 1), ("bn", "c1_bn", 8), ("relu",),
            ("conv", "c2", 8, 16, 3, 1, 1), ("bn", "c2_bn", 16), ("relu",), ("maxpool", 2, 0, 2),
            ("conv", "c3", 16, 16, 3, 1, 1), ("bn", "c3_bn", 16), ("relu",), ("maxpool", 2, 0, 2),
            ("flatten",), ("fc", "f1", 16 * 4 * 4, 32), ("fc", "f2", 32, 10)]


@pytest.mark.parametrize("split,fuse", [(None, False), ({0: 4, 3: 4}, False), ({3: 3}, False), (None, True), ({0: 4, 3: 4}, True)])
def test_convnet_momentum_tracks_oracle_with_and_without_split(split, fuse):
    from tsplit_amd import ndarray, trainer
    rng = np.random.RandomState(7)
    spec = _small_convnet()
    X = rng.normal(size=(8, 3, 16, 16)).astype(np.float32)
    Y = _onehot(rng.randint(0, 10, 8), 10)
    params = trainer.init_params(spec, seed=5)
    ref_losses, ref_params = nets.train(spec, params, X, Y, steps=6, lr=0.05, momentum=0.9)
    ctx = ndarray.gpu(0)
    t = trainer.Trainer(spec, params, X.shape, 10, ctx, optimizer=("momentum", 0.05, 0.9), split=split,
                        fuse_bn_relu=fuse)
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for _ in range(6):
        t.step(gx, gy)
        losses.append(t.loss_value())
    rel = np.max(np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses))
    assert rel <= 1e-3, (rel, losses, ref_losses)
    for k in params:
        assert_close(t.params[k].asnumpy(), ref_params[k], 2e-3, k)


def _train_gpu(spec, params, X, Y, steps, opt, split=None, fuse=False, before_last=None):
    """`before_last`: a dict that receives the parameters and velocities as they are before the last step."""
    from tsplit_amd import ndarray, trainer
    ctx = ndarray.gpu(0)
    t = trainer.Trainer(spec, params, X.shape, Y.shape[1], ctx, optimizer=opt, split=split, fuse_bn_relu=fuse)
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    losses = []
    for i in range(steps):
        if before_last is not None and i == steps - 1:
            before_last["params"] = {k: v.asnumpy() for k, v in t.params.items()}
            before_last["velocity"] = {k: v.asnumpy() for k, v in t.state.items()}
        t.step(gx, gy)
        losses.append(t.loss_value())
    return t, losses


_VGG_20 = {}


def _vgg_20_step_oracle():
    """Spec, data, seeded parameters and the oracle's 20-step run, computed once for both routings."""
    if not _VGG_20:
        from tsplit_amd import trainer
        rng = np.random.RandomState(11)
        spec = trainer.vgg16_spec(num_classes=10, in_hw=32, fc_width=512)
        X = rng.normal(size=(8, 3, 32, 32)).astype(np.float32)
        Y = _onehot(rng.randint(0, 10, 8), 10)
        params = trainer.init_params(spec, seed=3)
        ref_losses, ref_params = nets.train(spec, params, X, Y, steps=20, lr=VGG_20_STEP_LR, momentum=0.9)
        _, f32_params = nets.train(spec, params, X, Y, steps=20, lr=VGG_20_STEP_LR, momentum=0.9, dtype=np.float32)
        _VGG_20.update(spec=spec, X=X, Y=Y, params=params, ref_losses=ref_losses, ref_params=ref_params, f32_params=f32_params)
    return _VGG_20


@pytest.mark.parametrize("winograd", [None, "1"])
def test_vgg16_topology_20_steps_tracks_oracle(winograd, monkeypatch):
    """The full VGG-16 layer list (13 conv+BN+Relu at 64 ... 512 channels, 5 pools, 3 FC) at 32x32,
    batch 8, with the two largest-resolution blocks run as 2 micro-tensors: 20 momentum steps against
    the oracle.  The step size is the one under which this 8-image batch is learnt smoothly (the loss
    falls from 4.8 to 0.7 over the 20 steps; ten times larger and the batch is memorised within three
    updates, after which rounding differences decide the curve), so a wrong gradient or update shows in
    the curve; what the 20 updates changed in every parameter is compared as well.  Once as the library
    routes these small layers itself (direct kernels), once with every layer but the first forced
    through the Winograd routine in all three passes."""
    if winograd:
        monkeypatch.setenv("TSPLIT_CONV_WINOGRAD", winograd)
    o = _vgg_20_step_oracle()
    spec, params, ref_losses, ref_params = o["spec"], o["params"], o["ref_losses"], o["ref_params"]
    assert ref_losses[-1] < 0.5 * ref_losses[0], ref_losses       # the run does train
    conv_idx = [i for i, l in enumerate(spec) if l[0] == "conv"]
    before = {}
    t, losses = _train_gpu(spec, params, o["X"], o["Y"], 20, ("momentum", VGG_20_STEP_LR, 0.9),
                           split={i: 2 for i in conv_idx[:4]}, before_last=before)
    rel = np.abs(np.array(losses) - np.array(ref_losses)) / np.abs(ref_losses)
    assert np.max(rel) <= 1e-3, (rel, losses, ref_losses)
    # This run amplifies whatever differs (the oracle's own float32 run leaves its float64 run by 2e-7 of the loss at
    # the first step and by 2e-4 to 4e-4 at the last ones), so the last step is also held to the oracle without any
    # history: its loss from the parameters the device itself had before it.
    l_ref, _, _ = nets.forward_backward(spec, before["params"], o["X"], o["Y"], want_grads=False)
    assert abs(losses[-1] - l_ref) <= LAST_STEP_LOSS_BAR * abs(l_ref), (losses[-1], l_ref)
    assert losses[-1] < 0.5 * losses[0]
    for k in params:
        got = t.params[k].asnumpy()
        if np.any(params[k] != 0):                 # BatchNorm biases start at zero: their value IS the change
            assert_close(got, ref_params[k], 2e-3, k)
        # what the 20 updates changed, against the yardstick: the same 20 steps of the oracle in float32
        # arithmetic move away from its float64 run by `off_f32`; the device's fp32 run may be at most
        # YARDSTICK_FACTOR times as far.  Parameters are stored in fp32 on all three sides; one near 1 (the
        # BatchNorm scales) is stored in steps of 2^-23, which each of the 20 roundings may take differently,
        # hence the second term
        d_ref = ref_params[k].astype(np.float64) - params[k]
        off = float(np.linalg.norm(got.astype(np.float64) - ref_params[k]))
        off_f32 = float(np.linalg.norm(o["f32_params"][k].astype(np.float64) - ref_params[k]))
        bound = YARDSTICK_FACTOR * off_f32 + YARDSTICK_FLOOR * np.linalg.norm(d_ref) + \
            np.sqrt(d_ref.size) * 20 * 2.0 ** -24 * np.max(np.abs(params[k]))
        assert off <= bound, "change of %s: off by %.3e in norm, the float32 oracle by %.3e, bound %.3e" % (k, off, off_f32, bound)


def _rel_l2(got, ref):
    got, ref = np.asarray(got, np.float64).ravel(), np.asarray(ref, np.float64).ravel()
    return float(np.linalg.norm(got - ref) / max(np.linalg.norm(ref), 1e-300))


def test_vgg16_224_natural_routing_every_operator_against_oracle():
    """VGG-16 at the benchmark's resolution (224x224, 1000 classes, He init), batch 8 with the first
    four convolutions on 2 micro-tensors, routed by the library itself: at these sizes it sends the
    112x112 and 56x56 layers through the Winograd routine in all three passes (asserted through the
    routing query, so the test cannot silently run on the direct kernels) and cuts the direct layers'
    tiles between blocks as it does at batch 64.

    Every operator call of the step is checked where it stands: its output against the float64 oracle
    applied to the very inputs the call read on the device (forward, both convolution gradients,
    BatchNorm with its parameter gradients, Relu, max pooling, the three matrix products per FC layer,
    the loss, the momentum update), to the operator bars: 2e-3 for conv / matmul, 1e-4 for BatchNorm and
    the update, exact for Relu and pooling.  The calls run in a real step's order on one stream, sharing
    the library's scratch memory as they do in the benchmark.

    End to end, the loss is held to 1e-3 of the oracle's.  The end-to-end parameter gradients of this
    13-layer net at initialisation are not a stable function of rounding: which of two nearly equal
    activations a pooling window or a Relu passes the gradient to flips with the last bit.  How far
    fp32 arithmetic by itself moves them is measured here, not assumed: the oracle runs a second time
    in float32, and every parameter's gradient from the device must lie within YARDSTICK_FACTOR times
    that run's distance from the float64 gradient (norm-wise, plus the operator tolerance as a floor).
    The tight bars sit on the operators above."""
    from oracle import ops
    from tsplit_amd import gpu_links as L, ndarray, trainer
    from util import max_rel_err
    rng = np.random.RandomState(21)
    spec = trainer.vgg16_spec(num_classes=1000, in_hw=224)
    X = rng.standard_normal(size=(8, 3, 224, 224)).astype(np.float32)
    Y = _onehot(rng.randint(0, 1000, 8), 1000)
    params = trainer.init_params(spec, seed=9, scheme="he")
    # the routing the library chooses for this run
    for imgs, c, o, hw in ((4, 64, 128, 112), (4, 128, 128, 112), (8, 128, 256, 56), (8, 256, 256, 56)):
        assert L.conv_takes_winograd(imgs, c, o, hw, hw, 3, 1, 1)
        assert L.conv_takes_winograd(imgs, c, o, hw, hw, 3, 1, 1, filter_gradient=True)
        assert L.conv_takes_winograd(imgs, o, c, hw, hw, 3, 1, 1, data_gradient=True)
    assert L.conv_takes_winograd(4, 64, 64, 224, 224, 3, 1, 1)
    lr, mom, eps = 0.01, 0.9, 0.01
    conv_idx = [i for i, l in enumerate(spec) if l[0] == "conv"]
    ctx = ndarray.gpu(0)
    t = trainer.Trainer(spec, params, X.shape, 1000, ctx, optimizer=("momentum", lr, mom),
                        split={i: 2 for i in conv_idx[:4]}, bn_eps=eps)
    gx, gy = ndarray.array(X, ctx), ndarray.array(Y, ctx)
    t.forward(gx, gy)
    t.backward(gy)
    gpu_loss = t.loss_value()
    grads = {k: v.asnumpy() for k, v in t.grads.items()}

    worst = {}

    def check(kind, what, got, ref, tol):
        err = max_rel_err(got, ref)
        assert np.isfinite(np.asarray(got)).all(), what
        assert err <= tol, "%s: max relative error %.3e > %.1e" % (what, err, tol)
        worst[kind] = max(worst.get(kind, 0.0), err)

    for li, layer in enumerate(spec):
        a, out, g_out = t.acts[li].asnumpy(), t.acts[li + 1].asnumpy(), t.dacts[li + 1].asnumpy()
        g_in = t.dacts[li].asnumpy() if li > 0 else None
        kind = layer[0]
        if kind == "conv":
            _, name, cin, cout, k, pad, stride = layer
            w = params[name + "_weight"]
            check("conv", name + " forward", out, ops.conv2d(a, w, pad, pad, stride), 2e-3)
            check("conv", name + " filter gradient", grads[name + "_weight"],
                  ops.conv2d_grad_filter(a, g_out, w.shape, pad, pad, stride), 2e-3)
            if li > 0:
                check("conv", name + " data gradient", g_in, ops.conv2d_grad_data(w, g_out, a.shape, pad, pad, stride), 2e-3)
        elif kind == "bn":
            name = layer[1]
            scale, bias = params[name + "_scale"], params[name + "_bias"]
            check("bn", name + " forward", out, ops.batchnorm_forward(a, scale, bias, eps)[0], 1e-4)
            dx, ds, db = ops.batchnorm_backward(g_out, a, scale, eps)
            check("bn", name + " input gradient", g_in, dx, 1e-4)
            check("bn", name + " scale gradient", grads[name + "_scale"].reshape(-1), ds.reshape(-1), 1e-4)
            check("bn", name + " bias gradient", grads[name + "_bias"].reshape(-1), db.reshape(-1), 1e-4)
        elif kind == "relu":
            assert np.array_equal(out, ops.relu(a).astype(np.float32)), (li, "relu")
            assert np.array_equal(g_in, ops.relu_grad(a, g_out).astype(np.float32)), (li, "relu gradient")
        elif kind == "maxpool":
            _, k, pad, stride = layer
            assert np.array_equal(out, ops.max_pool(a, k, k, pad, stride).astype(np.float32)), (li, "max pool")
            assert np.array_equal(g_in, ops.max_pool_grad(a, g_out, k, k, pad, stride).astype(np.float32)), (li, "max pool gradient")
        elif kind == "flatten":
            assert np.array_equal(out, a.reshape(out.shape)) and np.array_equal(g_in, g_out.reshape(g_in.shape))
        elif kind == "fc":
            name = layer[1]
            w = params[name + "_weight"]
            check("matmul", name + " forward", out, ops.matmul(a, False, w, False), 2e-3)
            check("matmul", name + " weight gradient", grads[name + "_weight"], ops.matmul(a, True, g_out, False), 2e-3)
            check("matmul", name + " input gradient", g_in, ops.matmul(g_out, False, w, True), 2e-3)
    logits = t.acts[-1].asnumpy()
    check("loss", "softmax cross-entropy", np.array([gpu_loss]), ops.softmax_ce(logits, Y), 1e-4)
    check("loss", "softmax cross-entropy gradient", t.dacts[-1].asnumpy(), ops.softmax_ce_grad(logits, Y, np.ones(1)), 1e-4)
    # measured: Winograd layers ~1e-5, direct ~1e-6, BatchNorm ~2e-7
    assert worst["conv"] < 1e-4 and worst["bn"] < 1e-5 and worst["matmul"] < 1e-4, worst
    # the update, from the gradients the device holds
    t.update()
    t.sync()
    for k, p0 in params.items():
        p, v = ops.momentum_update(p0, grads[k], np.zeros_like(p0), lr, mom, False)
        check("update", k + " after the update", t.params[k].asnumpy(), p, 1e-4)
        check("update", k + " velocity", t.state[k].asnumpy(), v, 1e-4)
    # end to end
    loss0, _, ref_grads = nets.forward_backward(spec, params, X, Y, eps)
    assert abs(gpu_loss - loss0) <= 1e-3 * abs(loss0), (gpu_loss, loss0)
    _, _, f32_grads = nets.forward_backward(spec, params, X, Y, eps, dtype=np.float32)
    l2 = {k: _rel_l2(grads[k].reshape(g.shape), g) for k, g in ref_grads.items()}
    yard = {k: _rel_l2(f32_grads[k].reshape(g.shape), g) for k, g in ref_grads.items()}
    over = {k: (l2[k], yard[k]) for k in l2 if l2[k] > YARDSTICK_FACTOR * yard[k] + YARDSTICK_FLOOR}
    print("end-to-end gradients, relative L2 distance from the float64 oracle (device, float32 oracle):",
          sorted(((k, round(l2[k], 6), round(yard[k], 6)) for k in l2), key=lambda r: -r[1])[:8])
    print("largest ratio device / float32 oracle:", max(l2[k] / max(yard[k], 1e-300) for k in l2))
    assert not over, sorted(over.items(), key=lambda kv: -kv[1][0])[:8]
    for k in ("vgg_fc3_weight", "vgg_fc2_weight", "vgg_fc1_weight"):      # nothing between them and the loss flips
        assert_close(grads[k], ref_grads[k], 2e-3, "gradient of " + k)
