"""CPU oracle: whole training steps assembled from oracle/ops.py.

THIS IS TEST INFRASTRUCTURE (same rule as oracle/ops.py).

A network is a list of layer tuples, the same `spec` format the product-side
trainer consumes (the spec itself is plain data and is handed in by the caller):
    ("conv", name, Cin, Cout, k, pad, stride)   weight [Cout,Cin,k,k], no bias
    ("bn", name, C)                            scale/bias [1,C,1,1]
    ("relu",)
    ("maxpool", k, pad, stride)
    ("flatten",)
    ("fc", name, n_in, n_out)                  weight [n_in,n_out], no bias
The loss is softmax cross-entropy on the last activation.  The graph wiring
follows the reference's autodiff rules (gpu_ops/executor.py:160-196 and each
op's `gradient`): conv -> (grad_data, grad_filter); matmul -> two matmuls with
transposes (gpu_ops/MatrixMult.py:95-124); first-layer data gradient is never
evaluated; the adjoint is seeded with ones (executor.py:175).  Unlike the
reference's active BatchNorm module, which drops the scale/bias gradients
(gpu_ops/BatchNorm.py:86-93), scale and bias are trained here, as its
BatchNorm2 variant does (gpu_ops/BatchNorm2.py:106-114).
"""
import numpy as np

from . import ops


def param_shapes(spec):
    shapes = {}
    for layer in spec:
        if layer[0] == "conv":
            _, name, cin, cout, k, _, _ = layer
            shapes[name + "_weight"] = (cout, cin, k, k)
        elif layer[0] == "bn":
            _, name, c = layer
            shapes[name + "_scale"] = (1, c, 1, 1)
            shapes[name + "_bias"] = (1, c, 1, 1)
        elif layer[0] == "fc":
            _, name, n_in, n_out = layer
            shapes[name + "_weight"] = (n_in, n_out)
    return shapes


def forward_backward(spec, params, x, labels, eps=0.01, dtype=np.float64, want_grads=True):
    """Returns (loss scalar, logits, grads dict)."""
    acts = [ops._f(x, dtype)]
    for layer in spec:
        a = acts[-1]
        kind = layer[0]
        if kind == "conv":
            _, name, _, _, k, pad, stride = layer
            acts.append(ops.conv2d(a, params[name + "_weight"], pad, pad, stride, dtype))
        elif kind == "bn":
            _, name, _ = layer
            acts.append(ops.batchnorm_forward(a, params[name + "_scale"], params[name + "_bias"], eps, dtype)[0])
        elif kind == "relu":
            acts.append(ops.relu(a, dtype))
        elif kind == "maxpool":
            _, k, pad, stride = layer
            acts.append(ops.max_pool(a, k, k, pad, stride).astype(dtype))
        elif kind == "flatten":
            acts.append(a.reshape(a.shape[0], -1))
        elif kind == "fc":
            _, name, _, _ = layer
            acts.append(ops.matmul(a, False, params[name + "_weight"], False, dtype))
        else:
            raise ValueError(kind)
    logits = acts[-1]
    loss = ops.softmax_ce(logits, labels, dtype)
    grads = {}
    if not want_grads:
        return float(loss[0]), logits, grads
    g = ops.softmax_ce_grad(logits, labels, np.ones(1), dtype)
    for li in range(len(spec) - 1, -1, -1):
        layer = spec[li]
        a_in = acts[li]
        kind = layer[0]
        first = li == 0
        if kind == "conv":
            _, name, _, _, k, pad, stride = layer
            w = params[name + "_weight"]
            grads[name + "_weight"] = ops.conv2d_grad_filter(a_in, g, w.shape, pad, pad, stride, dtype)
            g = None if first else ops.conv2d_grad_data(w, g, a_in.shape, pad, pad, stride, dtype)
        elif kind == "bn":
            _, name, _ = layer
            g, ds, db = ops.batchnorm_backward(g, a_in, params[name + "_scale"], eps, dtype)
            grads[name + "_scale"] = ds.reshape(1, -1, 1, 1)
            grads[name + "_bias"] = db.reshape(1, -1, 1, 1)
        elif kind == "relu":
            g = ops.relu_grad(a_in, g, dtype)
        elif kind == "maxpool":
            _, k, pad, stride = layer
            g = ops.max_pool_grad(a_in, g, k, k, pad, stride, dtype)
        elif kind == "flatten":
            g = g.reshape(a_in.shape)
        elif kind == "fc":
            _, name, _, _ = layer
            w = params[name + "_weight"]
            grads[name + "_weight"] = ops.matmul(a_in, True, g, False, dtype)
            g = None if first else ops.matmul(g, False, w, True, dtype)
    return float(loss[0]), logits, grads


def train(spec, params, x, labels, steps, lr, momentum=None, eps=0.01, dtype=np.float64):
    """`steps` full-batch steps of SGD (momentum=None) or momentum SGD on the same
    batch; returns the loss before each update and the final params.  Parameters
    are re-rounded to float32 after every update, as the device stores them."""
    params = {k: np.asarray(v, np.float32) for k, v in params.items()}
    vel = {k: np.zeros_like(v) for k, v in params.items()}
    losses = []
    for _ in range(steps):
        loss, _, grads = forward_backward(spec, params, x, labels, eps, dtype)
        losses.append(loss)
        for k in params:
            if momentum is None:
                params[k] = ops.sgd_update(params[k], grads[k], lr, dtype).astype(np.float32)
            else:
                p, v = ops.momentum_update(params[k], grads[k], vel[k], lr, momentum, False, dtype)
                params[k], vel[k] = p.astype(np.float32), v.astype(np.float32)
    return losses, params
