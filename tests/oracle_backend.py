"""numpy backend for tsplit_amd.graph.Tape built on the CPU oracle (test infrastructure):
the same graph code then runs once through the C ABI and once through oracle/ops.py."""
import numpy as np

from oracle import ops as O


def _s(a):
    """Values are stored as float32, as the device stores them."""
    return np.ascontiguousarray(a, dtype=np.float32)


class OracleBackend(object):
    def from_numpy(self, a):
        return _s(a)

    def to_numpy(self, x):
        return np.asarray(x)

    def reshape(self, x, shape):
        return _s(x).reshape(shape)

    def conv2d(self, x, w, xs, ws, ph, pw, s):
        return _s(O.conv2d(x, w, ph, pw, s))

    def conv2d_grad_data(self, w, dy, xs, ph, pw, s):
        return _s(O.conv2d_grad_data(w, dy, xs, ph, pw, s))

    def conv2d_grad_filter(self, x, dy, ws, ph, pw, s):
        return _s(O.conv2d_grad_filter(x, dy, ws, ph, pw, s))

    def matmul(self, a, ta, b, tb, out_shape):
        return _s(O.matmul(a, ta, b, tb))

    def batch_matmul(self, a, ta, b, tb, out_shape):
        return _s(O.batch_matmul(a, ta, b, tb))

    def bn(self, x, gamma, beta, xs, eps):
        return _s(O.batchnorm_forward(x, gamma, beta, eps)[0])

    def bn_grad(self, dy, x, gamma, xs, eps):
        dx, dg, db = O.batchnorm_backward(dy, x, gamma, eps)
        return _s(dx), _s(dg).reshape(1, -1, 1, 1), _s(db).reshape(1, -1, 1, 1)

    def bn_relu(self, x, gamma, beta, xs, eps):
        y, mean, var = O.batchnorm_forward(x, gamma, beta, eps)
        return _s(O.relu(y)), mean, var

    def bn_relu_grad(self, dy, x, gamma, beta, mean, var, xs, eps):
        y = O.batchnorm_forward(x, gamma, beta, eps)[0]
        return self.bn_grad(O.relu_grad(y, dy), x, gamma, xs, eps)

    def relu(self, x, shape):
        return _s(O.relu(x))

    def relu_grad(self, x, dy, shape):
        return _s(O.relu_grad(x, dy))

    def max_pool(self, x, xs, k, pad, s):
        return _s(O.max_pool(x, k, k, pad, s))

    def max_pool_grad(self, x, y, dy, xs, k, pad, s):
        return _s(O.max_pool_grad(x, dy, k, k, pad, s))

    def avg_pool(self, x, xs, k, pad, s):
        return _s(O.avg_pool(x, k, k, pad, s))

    def avg_pool_grad(self, x, y, dy, xs, k, pad, s):
        return _s(O.avg_pool_grad(dy, xs, k, k, pad, s))

    def add(self, a, b, shape):
        return _s(O.add(a, b))

    def mul_const(self, a, c, shape):
        return _s(O.mul_const(a, c))

    def add_const(self, a, c, shape):
        return _s(O.add_const(a, c))

    def mul(self, a, b, shape):
        return _s(O.mul(a, b))

    def sigmoid(self, x, shape):
        return _s(O.sigmoid(x))

    def tanh(self, x, shape):
        return _s(O.tanh(x))

    def slice(self, x, begin, out_shape):
        return _s(O.slice_(x, begin, out_shape))

    def slice_grad(self, dy, begin, in_shape):
        return _s(O.slice_grad(dy, begin, in_shape))

    def broadcast_shape(self, x, out_shape):
        return _s(O.broadcast_shape(x, out_shape))

    def reduce_sum(self, x, axes, out_shape):
        return _s(O.reduce_sum(x, axes)).reshape(out_shape)

    def broadcast_to(self, x, out_shape):
        return _s(O.broadcast_to(x, out_shape))

    def reduce_sum_axis_zero(self, x, out_shape):
        return _s(O.reduce_sum_axis_zero(np.asarray(x).reshape((-1,) + tuple(out_shape))))

    def concat(self, a, b, out_shape, axis):
        return _s(O.concat(a, b, axis))

    def concat_grad(self, dout, in_shape, axis, idx):
        return _s(O.concat_grad(dout, in_shape, axis, idx))

    def transpose(self, x, perm, out_shape):
        return O.transpose(x, perm)

    def where(self, cond, a, b, shape):
        return _s(O.where(cond, a, b))

    def one_hot(self, ids, out_shape):
        return O.one_hot(ids, out_shape[-1])

    def embedding(self, table, ids, out_shape):
        return O.embedding_lookup(table, ids)

    def embedding_grad(self, dy, ids, table_shape):
        return _s(O.embedding_lookup_grad(dy, ids, table_shape))

    def zeros(self, shape):
        return np.zeros(shape, np.float32)

    def softmax_ce(self, logits, labels):
        return _s(O.softmax_ce(logits, labels)).reshape(1)

    def softmax_ce_grad(self, logits, labels, shape, seed=1.0):
        return _s(O.softmax_ce_grad(logits, labels, np.full(1, seed, np.float32)))

    # ---- batch micro-tensors: rows [i * n / pieces, (i + 1) * n / pieces) as a view, and a copy into one
    def piece(self, x, pieces, index):
        rows = x.shape[0] // pieces
        assert rows * pieces == x.shape[0]
        return x[index * rows:(index + 1) * rows]

    def assign(self, dst, src):
        dst[...] = src

    def empty(self, shape):
        return np.empty(tuple(int(v) for v in shape), np.float32)

    def sgd(self, p, g, lr):
        p[...] = _s(O.sgd_update(p, g, lr))

    def sync(self):
        pass
