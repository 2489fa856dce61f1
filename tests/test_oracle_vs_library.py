"""The oracle against an independent library implementation: PyTorch-CPU (float64 tensors,
autograd for every gradient).  None of these checks shares code or formulas with the oracle, so
a wrong sign, a transposed operand or a dropped term in either fails them.  Skipped when torch
cannot be imported."""
import numpy as np
import pytest

from oracle import nets
from oracle import ops as O

torch = pytest.importorskip("torch")
F = torch.nn.functional

CONV = [
    # N, C, H, W, O, kH, kW, ph, pw, stride
    (2, 3, 9, 8, 4, 3, 3, 1, 1, 1),
    (1, 2, 11, 11, 3, 7, 7, 3, 3, 2),
    (2, 2, 6, 9, 3, 1, 7, 0, 3, 1),
    (2, 4, 8, 8, 5, 1, 1, 0, 0, 2),
    (1, 3, 10, 10, 2, 3, 3, 0, 0, 2),
    (2, 2, 7, 7, 3, 5, 5, 2, 2, 3),
]


def _t(a, grad=False):
    return torch.tensor(np.asarray(a, np.float32).astype(np.float64), requires_grad=grad)


@pytest.mark.parametrize("case", CONV)
def test_conv_forward_and_both_gradients(case, rng):
    N, C, H, W, Oc, kH, kW, ph, pw, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = rng.normal(size=(Oc, C, kH, kW)).astype(np.float32)
    xt, wt = _t(x, True), _t(w, True)
    yt = F.conv2d(xt, wt, padding=(ph, pw), stride=s)
    y = O.conv2d(x, w, ph, pw, s)
    assert y.shape == tuple(yt.shape)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-10, atol=1e-10)
    dy = rng.normal(size=y.shape).astype(np.float32)
    yt.backward(_t(dy))
    np.testing.assert_allclose(O.conv2d_grad_data(w, dy, x.shape, ph, pw, s), xt.grad.numpy(), rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(O.conv2d_grad_filter(x, dy, w.shape, ph, pw, s), wt.grad.numpy(), rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("shape", [(4, 3, 5, 6), (2, 5, 7, 7), (8, 2, 1, 1)])
def test_batchnorm_forward_and_gradient(shape, rng):
    x = (rng.normal(size=shape) * 2 + 1).astype(np.float32)
    g = rng.normal(size=shape[1]).astype(np.float32)
    b = rng.normal(size=shape[1]).astype(np.float32)
    dy = rng.normal(size=shape).astype(np.float32)
    xt, gt, bt = _t(x, True), _t(g, True), _t(b, True)
    yt = F.batch_norm(xt, None, None, gt, bt, training=True, eps=0.01)
    y, mean, var = O.batchnorm_forward(x, g, b, 0.01)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-9, atol=1e-9)
    yt.backward(_t(dy))
    dx, dg, db = O.batchnorm_backward(dy, x, g, 0.01)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-8, atol=1e-9)
    np.testing.assert_allclose(dg, gt.grad.numpy(), rtol=1e-8, atol=1e-9)
    np.testing.assert_allclose(db, bt.grad.numpy(), rtol=1e-8, atol=1e-9)


@pytest.mark.parametrize("case", [(2, 3, 8, 8, 2, 0, 2), (1, 2, 9, 9, 3, 1, 2), (2, 2, 7, 7, 3, 0, 2)])
def test_max_pool_and_gradient_on_distinct_values(case, rng):
    N, C, H, W, k, pad, s = case
    x = rng.permutation(N * C * H * W).reshape(N, C, H, W).astype(np.float32)     # no ties
    xt = _t(x, True)
    yt = F.max_pool2d(xt, k, s, pad)
    y = O.max_pool(x, k, k, pad, s)
    np.testing.assert_array_equal(y, yt.detach().numpy())
    dy = rng.normal(size=y.shape).astype(np.float32)
    yt.backward(_t(dy))
    np.testing.assert_allclose(O.max_pool_grad(x, dy, k, k, pad, s), xt.grad.numpy(), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", [(2, 3, 8, 8, 2, 0, 2), (1, 2, 9, 9, 3, 1, 1), (2, 2, 7, 7, 7, 0, 7)])
def test_avg_pool_counts_padding(case, rng):
    N, C, H, W, k, pad, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    xt = _t(x, True)
    yt = F.avg_pool2d(xt, k, s, pad, count_include_pad=True)
    y = O.avg_pool(x, k, k, pad, s)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-12, atol=1e-12)
    dy = rng.normal(size=y.shape).astype(np.float32)
    yt.backward(_t(dy))
    np.testing.assert_allclose(O.avg_pool_grad(dy, x.shape, k, k, pad, s), xt.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_softmax_cross_entropy_and_gradient(rng):
    y = (rng.normal(size=(6, 11)) * 3).astype(np.float32)
    lab = np.eye(11, dtype=np.float32)[rng.randint(0, 11, 6)] * 0.9 + 0.1 / 11
    yt = _t(y, True)
    loss = -(_t(lab) * F.log_softmax(yt, dim=1)).sum(dim=1).mean()
    np.testing.assert_allclose(O.softmax_ce(y, lab)[0], float(loss.detach()), rtol=1e-12)
    (loss * 1.7).backward()
    np.testing.assert_allclose(O.softmax_ce_grad(y, lab, np.array([1.7], np.float32)), yt.grad.numpy(), rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(O.softmax(y), F.softmax(_t(y), dim=1).numpy(), rtol=1e-12)


def test_whole_net_loss_and_parameter_gradients(rng):
    """conv+BN+Relu x2, max pool, flatten, two FC layers: the oracle's hand-wired backward sweep
    against autograd through the library's operators."""
    spec = [("conv", "c1", 3, 6, 3, 1, 1), ("bn", "c1_bn", 6), ("relu",), ("conv", "c2", 6, 6, 3, 1, 1), ("bn", "c2_bn", 6),
            ("relu",), ("maxpool", 2, 0, 2), ("flatten",), ("fc", "f1", 6 * 4 * 4, 12), ("fc", "f2", 12, 5)]
    params = {n: rng.normal(scale=0.3, size=s).astype(np.float32) for n, s in nets.param_shapes(spec).items()}
    x = rng.normal(size=(4, 3, 8, 8)).astype(np.float32)
    lab = np.eye(5, dtype=np.float32)[rng.randint(0, 5, 4)]
    loss, _, grads = nets.forward_backward(spec, params, x, lab, eps=0.01)
    P = {k: _t(v, True) for k, v in params.items()}
    h = _t(x)
    for layer in spec:
        kind = layer[0]
        if kind == "conv":
            h = F.conv2d(h, P[layer[1] + "_weight"], padding=layer[5], stride=layer[6])
        elif kind == "bn":
            h = F.batch_norm(h, None, None, P[layer[1] + "_scale"].reshape(-1), P[layer[1] + "_bias"].reshape(-1),
                             training=True, eps=0.01)
        elif kind == "relu":
            h = F.relu(h)
        elif kind == "maxpool":
            h = F.max_pool2d(h, layer[1], layer[3], layer[2])
        elif kind == "flatten":
            h = h.reshape(h.shape[0], -1)
        elif kind == "fc":
            h = h @ P[layer[1] + "_weight"]
    lt = -(_t(lab) * F.log_softmax(h, dim=1)).sum(dim=1).mean()
    lt.backward()
    # the oracle rounds every operator's inputs to float32 (what the device holds): 1e-7-level differences
    assert abs(float(loss) - float(lt.detach())) <= 1e-6 * abs(float(lt.detach()))
    for k, v in grads.items():
        np.testing.assert_allclose(np.asarray(v).reshape(P[k].shape), P[k].grad.numpy(), rtol=1e-4, atol=1e-7, err_msg=k)
