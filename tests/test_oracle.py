"""Pins the CPU oracle (oracle/ops.py) against things the mathematics fixes:
brute-force loops, library routines, adjoint identities, finite differences,
closed forms and hand-computed vectors.  The reference ships no tests or golden
vectors for this path, so these checks are what anchors parity."""
import numpy as np
import pytest
import scipy.signal

from oracle import loops, ops

CONV_CASES = [
    # N, C, H, W, O, kH, kW, pad_h, pad_w, stride
    (2, 3, 6, 6, 4, 3, 3, 1, 1, 1),     # VGG-style same conv
    (1, 2, 7, 7, 3, 3, 3, 1, 1, 2),     # stride 2, exact
    (2, 2, 8, 8, 3, 3, 3, 1, 1, 2),     # stride 2, floors (ResNet 3x3/s2/p1 case)
    (1, 3, 9, 9, 2, 7, 7, 3, 3, 2),     # ResNet stem shape class
    (1, 2, 5, 8, 3, 1, 7, 0, 3, 1),     # Inception 1x7, asymmetric pad
    (1, 2, 8, 5, 3, 7, 1, 3, 0, 1),     # Inception 7x1
    (2, 4, 5, 5, 3, 1, 1, 0, 0, 1),     # 1x1
    (1, 2, 6, 6, 2, 3, 3, 0, 0, 1),     # valid
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_forward_matches_loops_and_definition(case, rng):
    N, C, H, W, O, kH, kW, ph, pw, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = rng.normal(size=(O, C, kH, kW)).astype(np.float32)
    y = ops.conv2d(x, w, ph, pw, s)
    np.testing.assert_allclose(y, loops.conv2d_direct(x, w, ph, pw, s), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(y, loops.conv2d_loops(x.astype(np.float64), w.astype(np.float64), ph, pw, s),
                               rtol=1e-12, atol=1e-12)
    np.testing.assert_array_equal(ops.im2col(x, kH, kW, ph, pw, s), loops.im2col_loops(x, kH, kW, ph, pw, s))


def test_conv_reduces_to_scipy_correlate2d(rng):
    x = rng.normal(size=(1, 3, 9, 11)).astype(np.float32)
    w = rng.normal(size=(2, 3, 3, 3)).astype(np.float32)
    y = ops.conv2d(x, w, 0, 0, 1)
    for o in range(2):
        ref = sum(scipy.signal.correlate2d(x[0, c].astype(np.float64), w[o, c].astype(np.float64), mode="valid")
                  for c in range(3))
        np.testing.assert_allclose(y[0, o], ref, rtol=1e-12, atol=1e-12)
    # "same" padding: correlate2d mode=same with odd kernel equals pad 1
    y1 = ops.conv2d(x, w, 1, 1, 1)
    ref = sum(scipy.signal.correlate2d(x[0, c].astype(np.float64), w[1, c].astype(np.float64), mode="same")
              for c in range(3))
    np.testing.assert_allclose(y1[0, 1], ref, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("case", CONV_CASES)
def test_conv_backward_matches_loops_and_adjoint(case, rng):
    N, C, H, W, O, kH, kW, ph, pw, s = case
    x = rng.normal(size=(N, C, H, W)).astype(np.float32)
    w = rng.normal(size=(O, C, kH, kW)).astype(np.float32)
    y = ops.conv2d(x, w, ph, pw, s)
    dy = rng.normal(size=y.shape).astype(np.float32)
    dx = ops.conv2d_grad_data(w, dy, x.shape, ph, pw, s)
    dw = ops.conv2d_grad_filter(x, dy, w.shape, ph, pw, s)
    x64, w64, dy64 = x.astype(np.float64), w.astype(np.float64), dy.astype(np.float64)
    np.testing.assert_allclose(dx, loops.conv2d_grad_data_loops(w64, dy64, x.shape, ph, pw, s), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dw, loops.conv2d_grad_filter_loops(x64, dy64, w.shape, ph, pw, s), rtol=1e-12, atol=1e-12)
    # <conv(x,w),dy> = <x,bwd_data(w,dy)> = <w,bwd_filter(x,dy)>
    lhs = np.sum(y * dy64)
    np.testing.assert_allclose(np.sum(x64 * dx), lhs, rtol=1e-10)
    np.testing.assert_allclose(np.sum(w64 * dw), lhs, rtol=1e-10)


def test_matmul_transposes(rng):
    A = rng.normal(size=(5, 7)).astype(np.float32)
    B = rng.normal(size=(7, 3)).astype(np.float32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(ops.matmul(A, False, B, False), ref)
    np.testing.assert_allclose(ops.matmul(A.T.copy(), True, B, False), ref)
    np.testing.assert_allclose(ops.matmul(A, False, B.T.copy(), True), ref)
    np.testing.assert_allclose(ops.matmul(A.T.copy(), True, B.T.copy(), True), ref)
    # 2x2 known answer
    np.testing.assert_array_equal(ops.matmul([[1, 2], [3, 4]], False, [[5, 6], [7, 8]], False), [[19, 22], [43, 50]])


def test_batchnorm_forward_closed_form_and_invariants(rng):
    x = (rng.normal(size=(4, 3, 5, 6)) * 3 + 2).astype(np.float32)
    g = rng.normal(size=(1, 3, 1, 1)).astype(np.float32)
    b = rng.normal(size=(1, 3, 1, 1)).astype(np.float32)
    eps = 0.01
    y, mean, var = ops.batchnorm_forward(x, g, b, eps)
    for c in range(3):
        xc = x[:, c].astype(np.float64).ravel()
        mu = sum(xc) / len(xc)
        v = sum((xc - mu) ** 2) / len(xc)             # biased
        assert abs(mean[c] - mu) < 1e-12 and abs(var[c] - v) < 1e-12
        ref = float(g[0, c, 0, 0]) * (x[:, c].astype(np.float64) - mu) / np.sqrt(v + eps) + float(b[0, c, 0, 0])
        np.testing.assert_allclose(y[:, c], ref, rtol=1e-12, atol=1e-12)
        # invariants: mean(y) = beta ; var(y) = gamma^2 var/(var+eps)
        np.testing.assert_allclose(y[:, c].mean(), b[0, c, 0, 0], atol=1e-12)
        np.testing.assert_allclose(y[:, c].var(), float(g[0, c, 0, 0]) ** 2 * v / (v + eps), rtol=1e-12)


def test_batchnorm_backward_finite_differences(rng):
    x = rng.normal(size=(3, 2, 3, 2))
    g = rng.normal(size=(1, 2, 1, 1))
    b = rng.normal(size=(1, 2, 1, 1))
    dy = rng.normal(size=x.shape)
    # use values exactly representable in fp32 so that _f() rounding is a no-op
    x, g, b, dy = [a.astype(np.float32).astype(np.float64) for a in (x, g, b, dy)]
    eps = 0.01

    def f64(xx, gg, bb):
        D = xx.shape[1]
        mu = xx.mean(axis=(0, 2, 3)).reshape(1, D, 1, 1)
        v = xx.var(axis=(0, 2, 3)).reshape(1, D, 1, 1)
        return np.sum((gg * (xx - mu) / np.sqrt(v + eps) + bb) * dy)

    dx, dg, db = ops.batchnorm_backward(dy, x, g, eps)
    h = 1e-6
    num = np.zeros_like(x)
    for idx in np.ndindex(*x.shape):
        xp, xm = x.copy(), x.copy()
        xp[idx] += h
        xm[idx] -= h
        num[idx] = (f64(xp, g, b) - f64(xm, g, b)) / (2 * h)
    np.testing.assert_allclose(dx, num, rtol=1e-6, atol=1e-8)
    for c in range(2):
        e = np.zeros_like(g)
        e[0, c, 0, 0] = h
        np.testing.assert_allclose(dg[c], (f64(x, g + e, b) - f64(x, g - e, b)) / (2 * h), rtol=1e-6, atol=1e-8)
        np.testing.assert_allclose(db[c], (f64(x, g, b + e) - f64(x, g, b - e)) / (2 * h), rtol=1e-6, atol=1e-8)
    # invariant: dx sums to zero per channel; sum(dx * xhat) = 0 per channel
    np.testing.assert_allclose(dx.sum(axis=(0, 2, 3)), 0, atol=1e-12)


def test_relu_and_grad_special_cases():
    x = np.array([-2.0, -0.0, 0.0, 3.0], dtype=np.float32)
    dy = np.array([10.0, 20.0, 30.0, 40.0], dtype=np.float32)
    np.testing.assert_array_equal(ops.relu(x), [0, 0, 0, 3])
    np.testing.assert_array_equal(ops.relu_grad(x, dy), [0, 10, 15, 40])   # 0.5*dy at x == 0


POOL_CASES = [(2, 2, 0, 2, 6, 6), (3, 3, 1, 2, 7, 7), (3, 3, 0, 2, 7, 9), (3, 3, 1, 2, 8, 8), (2, 3, 0, 1, 5, 6)]


@pytest.mark.parametrize("kH,kW,pad,stride,H,W", POOL_CASES)
def test_maxpool_matches_loops_with_ties(kH, kW, pad, stride, H, W, rng):
    # few distinct values => many ties inside windows
    x = rng.randint(0, 3, size=(2, 3, H, W)).astype(np.float32)
    out, arg = loops.max_pool_loops(x, kH, kW, pad, stride)
    np.testing.assert_array_equal(ops.max_pool_argmax(x, kH, kW, pad, stride), arg)
    np.testing.assert_array_equal(ops.max_pool(x, kH, kW, pad, stride), out)
    dy = rng.normal(size=out.shape).astype(np.float32)
    np.testing.assert_array_equal(ops.max_pool_grad(x, dy, kH, kW, pad, stride, dtype=np.float32),
                                  loops.max_pool_grad_loops(x, dy, kH, kW, pad, stride))


def test_maxpool_constructed_ties():
    # all-equal window => top-left wins
    x = np.ones((1, 1, 4, 4), dtype=np.float32)
    np.testing.assert_array_equal(ops.max_pool_argmax(x, 2, 2, 0, 2)[0, 0], [[0, 2], [8, 10]])
    # overlapping 3x3/s2 windows sharing one maximum accumulate both gradients
    x = np.zeros((1, 1, 5, 5), dtype=np.float32)
    x[0, 0, 2, 2] = 5
    dy = np.array([[[[1, 2], [3, 4]]]], dtype=np.float32)
    dx = ops.max_pool_grad(x, dy, 3, 3, 0, 2)
    assert dx[0, 0, 2, 2] == 10 and dx.sum() == 10
    # padding never wins: negative inputs with pad 1
    x = -np.ones((1, 1, 4, 4), dtype=np.float32)
    assert (ops.max_pool(x, 3, 3, 1, 2) == -1).all()


def test_softmax_ce_closed_forms(rng):
    C = 7
    y = np.full((5, C), 3.25, dtype=np.float32)
    lab = np.eye(C, dtype=np.float32)[rng.randint(0, C, 5)]
    np.testing.assert_allclose(ops.softmax_ce(y, lab), [np.log(C)], rtol=1e-12)       # uniform logits
    y = rng.normal(size=(5, C)).astype(np.float32)
    sm = ops.softmax(y)
    np.testing.assert_allclose(sm.sum(axis=1), 1, rtol=1e-12)
    ref = np.mean([-np.log(sm[i, np.argmax(lab[i])]) for i in range(5)])
    np.testing.assert_allclose(ops.softmax_ce(y, lab)[0], ref, rtol=1e-12)
    # literal reference form log(softmax) agrees
    np.testing.assert_allclose(ops.softmax_ce(y, lab), np.mean(-np.sum(lab * np.log(sm), axis=1), keepdims=True), rtol=1e-12)
    g = ops.softmax_ce_grad(y, lab, np.array([2.0], dtype=np.float32))
    np.testing.assert_allclose(g.sum(axis=1), 0, atol=1e-12)                           # one-hot => rows sum to 0
    np.testing.assert_allclose(g, (sm - lab) * 2.0 / 5, rtol=1e-12)
    # finite difference of the loss
    h = 1e-6
    y64 = y.astype(np.float64)
    for idx in [(0, 0), (3, 4)]:
        yp, ym = y64.copy(), y64.copy()
        yp[idx] += h
        ym[idx] -= h
        f = lambda z: np.mean(-np.sum(lab * (z - np.log(np.sum(np.exp(z), axis=1, keepdims=True))), axis=1))
        np.testing.assert_allclose(g[idx] / 2.0, (f(yp) - f(ym)) / (2 * h), rtol=1e-5, atol=1e-9)


def test_optimizers_hand_computed():
    p, g = np.array([1.0], np.float32), np.array([0.5], np.float32)
    assert ops.sgd_update(p, g, 0.5)[0] == 0.75
    # momentum 0.5, lr 0.5, g = 0.5 constant: v: -0.25, -0.375, -0.4375 ; p: 0.75, 0.375, -0.0625
    v = np.zeros(1, np.float32)
    ps = []
    for _ in range(3):
        p, v = ops.momentum_update(p, g, v, 0.5, 0.5)
        ps.append(float(p[0]))
    assert ps == [0.75, 0.375, -0.0625] and float(v[0]) == -0.4375
    # nesterov, same numbers: v1 = .5*(0-.25) = -.125, p1 = 1-.125-.25 = .625 ; v2 = .5*(-.125-.25) = -.1875, p2 = .625-.1875-.25 = .1875
    p, v = np.array([1.0], np.float32), np.zeros(1, np.float32)
    p, v = ops.momentum_update(p, g, v, 0.5, 0.5, True)
    assert float(p[0]) == 0.625 and float(v[0]) == -0.125
    p, v = ops.momentum_update(p, g, v, 0.5, 0.5, True)
    assert float(p[0]) == 0.1875 and float(v[0]) == -0.1875
    # adagrad: acc = 4, p = 1 - 0.5*2/(2+0) = 0.5
    p, acc = ops.adagrad_update(np.array([1.0]), np.array([2.0]), np.zeros(1), 0.5, 0.0)
    assert float(p[0]) == 0.5 and float(acc[0]) == 4.0
    # adam step 1 with eps=0: bias-corrected m = g, v = g^2 => p -= lr*sign(g)
    b1, b2 = 0.9, 0.999
    p, m, vv = ops.adam_update(np.array([1.0]), np.array([0.5]), np.zeros(1), np.zeros(1), 0.25, b1, b2, b1, b2, 0.0)
    np.testing.assert_allclose(p, [0.75], rtol=1e-12)
    np.testing.assert_allclose(m, [0.05], rtol=1e-12)
    np.testing.assert_allclose(vv, [0.00025], rtol=1e-12)
    # step 2 with g = -0.5: m = .9*.05 - .05 = -.005; v = .999*.00025 + .00025 = .00049975
    p, m, vv = ops.adam_update(p, np.array([-0.5]), m, vv, 0.25, b1, b2, b1 * b1, b2 * b2, 0.0)
    mc, vc = -0.005 / (1 - 0.81), 0.00049975 / (1 - 0.998001)
    # state was re-rounded to float32 between the steps (the device stores fp32), hence 1e-6
    np.testing.assert_allclose(p, [0.75 - 0.25 * mc / np.sqrt(vc)], rtol=1e-6)


def test_split_arithmetic():
    assert ops.split_shape((10, 3, 2, 2), 4) == [(3, 3, 2, 2), (3, 3, 2, 2), (2, 3, 2, 2), (2, 3, 2, 2)]
    offs = [ops.micro_tensor_view((10, 3, 2, 2), 4, i)[0] for i in range(4)]
    assert offs == [0, 36, 72, 96]
    x = np.arange(10 * 12, dtype=np.float32).reshape(10, 3, 2, 2)
    pieces = []
    for i in range(4):
        off, shp = ops.micro_tensor_view(x.shape, 4, i)
        pieces.append(x.ravel()[off:off + int(np.prod(shp))].reshape(shp))
    np.testing.assert_array_equal(np.concatenate(pieces, axis=0), x)       # views tile the parent exactly
    for a, b in zip(pieces, np.array_split(x, 4, axis=0)):
        np.testing.assert_array_equal(a, b)
    assert ops.micro_tensor_view((64, 64, 224, 224), 4, 3) == (3 * 16 * 64 * 224 * 224, (16, 64, 224, 224))
    # channel "split" relabels a contiguous chunk
    assert ops.micro_tensor_view((1, 6, 2, 2), 4, 2, 1) == (16, (1, 1, 2, 2))
    # overlapped buffer: out 8 elems, in 16 elems in 4 pieces, 1 overlapping
    assert ops.reuse_alloc_layout((16,), (8,), 4, 1) == (32 + 48, 16, 0)


def test_concat_slice(rng):
    a = rng.normal(size=(2, 3, 4)).astype(np.float32)
    b = rng.normal(size=(2, 5, 4)).astype(np.float32)
    c = ops.concat(a, b, 1)
    assert c.shape == (2, 8, 4)
    np.testing.assert_array_equal(ops.concat_grad(c, a.shape, 1, 0), a)
    np.testing.assert_array_equal(ops.concat_grad(c, b.shape, 1, 1), b)
    s = ops.slice_(c, (1, 2, 1), (1, 4, 2))
    np.testing.assert_array_equal(s, c[1:2, 2:6, 1:3])
    gs = ops.slice_grad(s, (1, 2, 1), c.shape)
    assert gs.sum() == s.sum() and gs[1, 2, 1] == s[0, 0, 0] and gs[0].sum() == 0
