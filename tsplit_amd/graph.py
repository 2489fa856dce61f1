"""A small reverse-mode tape over the operator library, for graphs with branches.

The reference builds such graphs with `ad.<op>_op` nodes and differentiates them with
`ad.gradients` (python/athena/gpu_ops/executor.py:160-196); each node's `compute` calls one
`gpu_links` function and its `gradient` names the nodes of the backward pass.  This tape does
the same work eagerly: every method below runs one forward operator and records the calls of
the backward operators the reference's `gradient` would schedule (cited per method).  It
exists so that the residual, multi-branch and attention graphs of the reference's examples
can be run through the C ABI; `trainer.py` remains the harness of the sequential nets.

The arithmetic comes from a backend object.  `GpuBackend` (below) maps every primitive onto
`gpu_links`; the tests plug in a numpy backend with the same methods to check whole graphs.
"""
import numpy as np

from . import gpu_links as L
from . import ndarray


class Var(object):
    """A value on the tape: backend array, shape, accumulated gradient; `node` is the index of the
    operator call that produced it on its tape (-1 for parameters, inputs and constants)."""
    __slots__ = ["value", "shape", "grad", "needs_grad", "name", "node"]

    def __init__(self, value, shape, needs_grad, name=None):
        self.value, self.shape, self.grad, self.needs_grad, self.name = value, tuple(shape), None, needs_grad, name
        self.node = -1


class Node(object):
    """One operator call: its output, the closure of its backward operators (None when no input
    needs a gradient), the Vars it read and the Vars its backward closure reads again."""
    __slots__ = ["out", "back", "inputs", "saved", "index", "redo"]

    def __init__(self, out, back, inputs, saved, index, redo=None):
        self.out, self.back, self.inputs, self.saved, self.index = out, back, tuple(inputs), tuple(saved), index
        # for operators that are cheap to run again (one to three passes over HBM): a closure that
        # computes the output once more from the inputs' current values, with the same bits
        self.redo = redo


SELF = object()      # in a `saved` list: the operator's own output


def _prod(shape):
    n = 1
    for s in shape:
        n *= int(s)
    return n


def conv_out(size, k, pad, stride):
    return (size + 2 * pad - k) // stride + 1


class GpuBackend(object):
    """Primitives on device arrays, one `gpu_links` call each (plus the output allocation)."""

    L = L        # the links module; a subclass that only counts memory puts a stand-in here

    def __init__(self, ctx=None, stream=None):
        self.ctx = ctx or ndarray.gpu(0)
        self.stream = stream

    # ---- batch micro-tensors
    def piece(self, x, pieces, index):
        """Rows [index * n / pieces, (index + 1) * n / pieces) of x as a zero-copy view
        (DLArraySliceForMicroTensor along the batch)."""
        return ndarray.slice_for_micro_tensor(x, index, pieces)

    def assign(self, dst, src):
        """dst <- src on the compute stream (dst is usually a micro-tensor view)."""
        src.copyto(dst, self.stream)

    # ---- storage
    def from_numpy(self, a):
        return ndarray.array(np.ascontiguousarray(a, dtype=np.float32), self.ctx)

    def to_numpy(self, x):
        return x.asnumpy()

    def empty(self, shape):
        return ndarray.empty(tuple(int(s) for s in shape), self.ctx)

    def reshape(self, x, shape):
        out = self.empty(shape)
        self.L.array_reshape(x, out, self.stream)
        return out

    # ---- contractions
    def conv2d(self, x, w, xs, ws, ph, pw, s):
        y = self.empty((xs[0], ws[0], conv_out(xs[2], ws[2], ph, s), conv_out(xs[3], ws[3], pw, s)))
        L.CuDNN_conv2d(x, w, y, ph, pw, s, self.stream)
        return y

    def conv2d_grad_data(self, w, dy, xs, ph, pw, s):
        dx = self.empty(xs)
        L.CuDNN_conv2d_gradient_of_data(w, dy, dx, ph, pw, s, self.stream)
        return dx

    def conv2d_grad_filter(self, x, dy, ws, ph, pw, s):
        dw = self.empty(ws)
        L.CuDNN_conv2d_gradient_of_filter(x, dy, dw, ph, pw, s, self.stream)
        return dw

    def matmul(self, a, ta, b, tb, out_shape):
        c = self.empty(out_shape)
        self.L.matrix_multiply(a, ta, b, tb, c, self.stream)
        return c

    def batch_matmul(self, a, ta, b, tb, out_shape):
        c = self.empty(out_shape)
        self.L.batch_matrix_multiply(a, ta, b, tb, c, self.stream)
        return c

    # ---- normalisation, activations, pooling
    def bn(self, x, gamma, beta, xs, eps):
        y = self.empty(xs)
        self.L.CuDNN_Batch_Normalization(x, gamma, beta, y, None, None, 0.99, eps, self.stream)
        return y

    def bn_grad(self, dy, x, gamma, xs, eps):
        dx, dg, db = self.empty(xs), self.empty((1, xs[1], 1, 1)), self.empty((1, xs[1], 1, 1))
        self.L.CuDNN_Batch_Normalization_gradient(dy, x, gamma, dx, dg, db, None, None, eps, self.stream)
        return dx, dg, db

    def bn_relu(self, x, gamma, beta, xs, eps):
        """-> (relu(bn(x)), saved mean, saved inverse deviation): one call, the BatchNorm output is never written."""
        y, mean, istd = self.empty(xs), self.empty((1, xs[1], 1, 1)), self.empty((1, xs[1], 1, 1))
        self.L.batch_norm_relu(x, gamma, beta, y, mean, istd, eps, stream=self.stream)
        return y, mean, istd

    def bn_relu_grad(self, dy, x, gamma, beta, mean, istd, xs, eps):
        dx, dg, db = self.empty(xs), self.empty((1, xs[1], 1, 1)), self.empty((1, xs[1], 1, 1))
        self.L.batch_norm_relu_gradient(dy, x, gamma, beta, dx, dg, db, mean, istd, eps, stream=self.stream)
        return dx, dg, db

    def relu(self, x, shape):
        y = self.empty(shape)
        self.L.relu(x, y, self.stream)
        return y

    def relu_grad(self, x, dy, shape):
        dx = self.empty(shape)
        self.L.relu_gradient(x, dy, dx, self.stream)
        return dx

    def max_pool(self, x, xs, k, pad, s):
        y = self.empty((xs[0], xs[1], conv_out(xs[2], k, pad, s), conv_out(xs[3], k, pad, s)))
        L.CuDNN_max_pooling2d(x, k, k, y, pad, s, self.stream)
        return y

    def max_pool_grad(self, x, y, dy, xs, k, pad, s):
        dx = self.empty(xs)
        L.CuDNN_max_pooling2d_gradient(y, dy, x, k, k, dx, pad, s, self.stream)
        return dx

    def avg_pool(self, x, xs, k, pad, s):
        y = self.empty((xs[0], xs[1], conv_out(xs[2], k, pad, s), conv_out(xs[3], k, pad, s)))
        L.CuDNN_average_pooling2d(x, k, k, y, pad, s, self.stream)
        return y

    def avg_pool_grad(self, x, y, dy, xs, k, pad, s):
        dx = self.empty(xs)
        L.CuDNN_average_pooling2d_gradient(y, dy, x, k, k, dx, pad, s, self.stream)
        return dx

    # ---- elementwise, broadcast, reduce, layout
    def add(self, a, b, shape):
        c = self.empty(shape)
        self.L.matrix_elementwise_add(a, b, c, self.stream)
        return c

    def mul_const(self, a, c, shape):
        out = self.empty(shape)
        self.L.matrix_elementwise_multiply_by_const(a, c, out, self.stream)
        return out

    def add_const(self, a, c, shape):
        out = self.empty(shape)
        self.L.matrix_elementwise_add_by_const(a, c, out, self.stream)
        return out

    def mul(self, a, b, shape):
        out = self.empty(shape)
        self.L.matrix_elementwise_multiply(a, b, out, self.stream)
        return out

    def sigmoid(self, x, shape):
        out = self.empty(shape)
        self.L.sigmoid(x, out, self.stream)
        return out

    def tanh(self, x, shape):
        out = self.empty(shape)
        self.L.tanh(x, out, self.stream)
        return out

    def slice(self, x, begin, out_shape):
        out = self.empty(out_shape)
        self.L.matrix_slice(x, out, begin, self.stream)
        return out

    def slice_grad(self, dy, begin, in_shape):
        out = self.empty(in_shape)
        self.L.matrix_slice_gradient(dy, out, begin, self.stream)
        return out

    def broadcast_shape(self, x, out_shape):
        out = self.empty(out_shape)
        self.L.broadcast_shape(x, out, None, self.stream)
        return out

    def reduce_sum(self, x, axes, out_shape):
        out = self.empty(out_shape)
        self.L.reduce_sum(x, out, axes, self.stream)
        return out

    def broadcast_to(self, x, out_shape):
        out = self.empty(out_shape)
        self.L.broadcast_to(x, out, self.stream)
        return out

    def reduce_sum_axis_zero(self, x, out_shape):
        out = self.empty(out_shape)
        self.L.reduce_sum_axis_zero(x, out, self.stream)
        return out

    def concat(self, a, b, out_shape, axis):
        out = self.empty(out_shape)
        self.L.concat(a, b, out, axis, self.stream)
        return out

    def concat_grad(self, dout, in_shape, axis, idx):
        g = self.empty(in_shape)
        self.L.concat_gradient(dout, g, axis, idx, self.stream)
        return g

    def transpose(self, x, perm, out_shape):
        out = self.empty(out_shape)
        self.L.matrix_transpose(x, out, perm, self.stream)
        return out

    def where(self, cond, a, b, shape):
        out = self.empty(shape)
        self.L.where(cond, a, b, out, self.stream)
        return out

    def one_hot(self, ids, out_shape):
        out = self.empty(out_shape)
        self.L.one_hot(ids, out, self.stream)
        return out

    def embedding(self, table, ids, out_shape):
        out = self.empty(out_shape)
        self.L.embedding_lookup(table, ids, out, self.stream)
        return out

    def embedding_grad(self, dy, ids, table_shape):
        g = self.empty(table_shape)
        self.L.embedding_lookup_gradient(dy, ids, g, self.stream)
        return g

    def zeros(self, shape):
        out = self.empty(shape)
        self.L.array_set(out, 0.0, self.stream)
        return out

    # ---- loss, update
    def softmax_ce(self, logits, labels):
        loss = self.empty((1,))
        self.L.softmax_cross_entropy(logits, labels, loss, self.stream)
        return loss

    def softmax_ce_grad(self, logits, labels, shape, seed=1.0):
        one = self.empty((1,))
        self.L.array_set(one, float(seed), self.stream)
        g = self.empty(shape)
        self.L.softmax_cross_entropy_gradient(logits, labels, one, g, self.stream)
        return g

    def sgd(self, p, g, lr):
        self.L.sgd_update(p, g, lr, self.stream)

    def sync(self):
        if self.stream:
            self.stream.sync()
        else:
            ndarray.empty((1,), self.ctx).asnumpy()


def _op(fn):
    """Marks an operator method of Tape: every call goes through Tape._call, so that a tape may log the
    calls of a builder (trace) or put them off and run them per batch micro-tensor (MicroTape)."""
    def call(self, *args, **kwargs):
        return self._call(fn, args, kwargs)
    call.__name__, call.__doc__ = fn.__name__, fn.__doc__
    return call


class Tape(object):
    # the builders' BatchNorm + Relu pairs as one node each (bn_then_relu); off: the reference's two nodes
    fuse_bn_relu = False

    def __init__(self, backend):
        self.b = backend
        self._nodes = []     # every operator call, in order (Node)
        self._log = None     # with a list here, every operator call is appended as (name, args, kwargs)

    def _call(self, fn, args, kwargs):
        if self._log is not None:
            self._log.append((fn.__name__, args, kwargs))
        return fn(self, *args, **kwargs)

    # ---- leaves
    def param(self, value, shape, name=None):
        return Var(value, shape, True, name)

    def const(self, value, shape, name=None):
        return Var(value, shape, False, name)

    def _out(self, value, shape, inputs, backward, saved=None, redo=None):
        """Registers an operator call.  `saved`: the Vars the backward closure reads (SELF for the
        output itself); by default the inputs.  A closure must read them as `var.value` when it
        runs, so that an executor may move a value off the device in between.  `redo`: see Node."""
        v = Var(value, shape, any(i.needs_grad for i in inputs))
        saved = inputs if saved is None else [v if s is SELF else s for s in saved]
        node = Node(v, backward if v.needs_grad else None, inputs, saved if v.needs_grad else (), len(self._nodes), redo)
        v.node = node.index
        self._nodes.append(node)
        self._after_forward(node)
        return v

    # hooks of executors that manage memory (tsplit_amd.tape_budget)
    def _after_forward(self, node):
        pass

    def _before_backward(self, node):
        pass

    def _after_backward(self, node):
        pass

    def _acc(self, var, g):
        if not var.needs_grad:
            return
        var.grad = g if var.grad is None else self.b.add(var.grad, g, var.shape)

    # ---- operators (reference gradient rules cited)
    @_op
    def conv2d(self, x, w, ph, pw, stride):
        """gpu_ops/Conv2d.py:100-118 (compute), :120 (gradient: a data-gradient and a filter-gradient node)."""
        y = self.b.conv2d(x.value, w.value, x.shape, w.shape, ph, pw, stride)
        ys = (x.shape[0], w.shape[0], conv_out(x.shape[2], w.shape[2], ph, stride), conv_out(x.shape[3], w.shape[3], pw, stride))

        def back(g):
            if w.needs_grad:
                self._acc(w, self.b.conv2d_grad_filter(x.value, g, w.shape, ph, pw, stride))
            if x.needs_grad:
                self._acc(x, self.b.conv2d_grad_data(w.value, g, x.shape, ph, pw, stride))
        return self._out(y, ys, [x, w], back, saved=[x, w])

    @_op
    def batch_norm(self, x, gamma, beta, eps=0.01):
        """gpu_ops/BatchNorm.py:54-83 (compute), :166-227 (gradient node; statistics recomputed, no
        saved arrays); gamma / beta receive their gradients as in gpu_ops/BatchNorm2.py:104-114."""
        def fwd():
            return self.b.bn(x.value, gamma.value, beta.value, x.shape, eps)

        def back(g):
            dx, dg, db = self.b.bn_grad(g, x.value, gamma.value, x.shape, eps)
            self._acc(x, dx)
            self._acc(gamma, dg)
            self._acc(beta, db)
        return self._out(fwd(), x.shape, [x, gamma, beta], back, saved=[x, gamma], redo=fwd)

    @_op
    def batch_norm_relu(self, x, gamma, beta, eps=0.01):
        """BatchNorm and the Relu behind it as one node (TSplit_BatchNormRelu / _gradient; the reference's graph
        has two nodes, gpu_ops/BatchNorm.py and gpu_ops/Relu.py): the BatchNorm output is never written, and
        the gradient reads the BatchNorm's input, the parameters and the two saved statistics vectors."""
        stats = [None, None]

        def fwd():
            r = self.b.bn_relu(x.value, gamma.value, beta.value, x.shape, eps)
            if r is None:                      # a backend that only records shapes
                return None
            y, stats[0], stats[1] = r
            return y

        def back(g):
            dx, dg, db = self.b.bn_relu_grad(g, x.value, gamma.value, beta.value, stats[0], stats[1], x.shape, eps)
            self._acc(x, dx)
            self._acc(gamma, dg)
            self._acc(beta, db)
        return self._out(fwd(), x.shape, [x, gamma, beta], back, saved=[x, gamma, beta], redo=fwd)

    def bn_then_relu(self, x, gamma, beta, eps=0.01):
        """The pair as the reference's graph has it (two nodes), or as one node when the tape was asked to fuse."""
        if self.fuse_bn_relu:
            return self.batch_norm_relu(x, gamma, beta, eps)
        return self.relu(self.batch_norm(x, gamma, beta, eps))

    @_op
    def relu(self, x):
        """gpu_ops/Relu.py:51,117."""
        def fwd():
            return self.b.relu(x.value, x.shape)
        return self._out(fwd(), x.shape, [x], lambda g: self._acc(x, self.b.relu_grad(x.value, g, x.shape)), redo=fwd)

    @_op
    def max_pool(self, x, k, pad, stride):
        """gpu_ops/MaxPool.py:119 (compute), :146 (gradient)."""
        y = self.b.max_pool(x.value, x.shape, k, pad, stride)
        ys = (x.shape[0], x.shape[1], conv_out(x.shape[2], k, pad, stride), conv_out(x.shape[3], k, pad, stride))
        out = None
        out = self._out(y, ys, [x], lambda g: self._acc(x, self.b.max_pool_grad(x.value, out.value, g, x.shape, k, pad, stride)),
                        saved=[x, SELF])
        return out

    @_op
    def avg_pool(self, x, k, pad, stride):
        """gpu_ops/AvgPool.py:78 (compute), :103-104 (gradient)."""
        y = self.b.avg_pool(x.value, x.shape, k, pad, stride)
        ys = (x.shape[0], x.shape[1], conv_out(x.shape[2], k, pad, stride), conv_out(x.shape[3], k, pad, stride))
        out = None
        out = self._out(y, ys, [x], lambda g: self._acc(x, self.b.avg_pool_grad(x.value, out.value, g, x.shape, k, pad, stride)),
                        saved=[x, SELF])
        return out

    @_op
    def add(self, a, b):
        """gpu_ops/AddElewise.py:54 (compute), :95 (gradient: both inputs receive the output gradient)."""
        assert a.shape == b.shape, (a.shape, b.shape)

        def fwd():
            return self.b.add(a.value, b.value, a.shape)

        def back(g):
            self._acc(a, g)
            self._acc(b, g)
        return self._out(fwd(), a.shape, [a, b], back, saved=[], redo=fwd)

    @_op
    def scale(self, a, c):
        """gpu_ops/MultiplyConst.py:45 (compute), :63 (gradient: the output gradient times the constant)."""
        def fwd():
            return self.b.mul_const(a.value, c, a.shape)
        return self._out(fwd(), a.shape, [a], lambda g: self._acc(a, self.b.mul_const(g, c, a.shape)), saved=[], redo=fwd)

    @_op
    def shift(self, a, c):
        def fwd():
            return self.b.add_const(a.value, c, a.shape)
        return self._out(fwd(), a.shape, [a], lambda g: self._acc(a, g), saved=[], redo=fwd)

    @_op
    def mul(self, a, b):
        """gpu_ops/MultiplyElewise.py (compute; gradient: each input receives the other times the
        output gradient)."""
        assert a.shape == b.shape, (a.shape, b.shape)

        def fwd():
            return self.b.mul(a.value, b.value, a.shape)

        def back(g):
            self._acc(a, self.b.mul(b.value, g, a.shape))
            self._acc(b, self.b.mul(a.value, g, a.shape))
        return self._out(fwd(), a.shape, [a, b], back, redo=fwd)

    @_op
    def sigmoid(self, x):
        """gpu_ops/Sigmoid.py:58-61: gradient s * (1 + -1 * s) * g, built from the same elementwise
        operators the reference's gradient graph uses."""
        y = self.b.sigmoid(x.value, x.shape)
        out = None

        def back(g):
            one_minus = self.b.add_const(self.b.mul_const(out.value, -1.0, x.shape), 1.0, x.shape)
            self._acc(x, self.b.mul(self.b.mul(out.value, one_minus, x.shape), g, x.shape))
        out = self._out(y, x.shape, [x], back, saved=[SELF])
        return out

    @_op
    def tanh(self, x):
        """gpu_ops/Tanh.py:59-61: gradient (1 + (-1 * t) * t) * g."""
        y = self.b.tanh(x.value, x.shape)
        out = None

        def back(g):
            d = self.b.add_const(self.b.mul(self.b.mul_const(out.value, -1.0, x.shape), out.value, x.shape), 1.0, x.shape)
            self._acc(x, self.b.mul(d, g, x.shape))
        out = self._out(y, x.shape, [x], back, saved=[SELF])
        return out

    @_op
    def slice(self, x, begin, size):
        """gpu_ops/Slice.py:47-81: tf.slice semantics, a size of -1 runs to the end; the gradient
        writes the output gradient into zeros at `begin` (:126-141)."""
        begin = tuple(int(v) for v in begin)
        shape = tuple(int(x.shape[d] - begin[d] if n == -1 else n) for d, n in enumerate(size))
        y = self.b.slice(x.value, begin, shape)
        return self._out(y, shape, [x], lambda g: self._acc(x, self.b.slice_grad(g, begin, x.shape)), saved=[])

    @_op
    def reshape(self, a, shape):
        """gpu_ops/Reshape.py:42 (compute: a copy), :61 (gradient: reshaped back)."""
        shape = list(shape)
        if -1 in shape:
            known = _prod([s for s in shape if s != -1])
            shape[shape.index(-1)] = _prod(a.shape) // known
        shape = tuple(shape)
        def fwd():
            return self.b.reshape(a.value, shape)
        return self._out(fwd(), shape, [a], lambda g: self._acc(a, self.b.reshape(g, a.shape)), saved=[], redo=fwd)

    @_op
    def concat(self, a, b, axis):
        """gpu_ops/Concat.py:47-60 (compute), :65 (gradient: two concat_gradient nodes, idx 0 and 1)."""
        shape = list(a.shape)
        shape[axis] += b.shape[axis]
        shape = tuple(shape)
        def fwd():
            return self.b.concat(a.value, b.value, shape, axis)
        y = fwd()

        def back(g):
            if a.needs_grad:
                self._acc(a, self.b.concat_grad(g, a.shape, axis, 0))
            if b.needs_grad:
                self._acc(b, self.b.concat_grad(g, b.shape, axis, 1))
        return self._out(y, shape, [a, b], back, saved=[], redo=fwd)

    @_op
    def matmul(self, a, b, trans_a=False, trans_b=False):
        """gpu_ops/MatrixMult.py:57-86 (compute), :95-124 (gradient)."""
        m = a.shape[1] if trans_a else a.shape[0]
        n = b.shape[0] if trans_b else b.shape[1]
        y = self.b.matmul(a.value, trans_a, b.value, trans_b, (m, n))

        def back(g):
            if a.needs_grad:
                if not trans_a:
                    ga = self.b.matmul(g, False, b.value, not trans_b, a.shape)
                else:
                    ga = self.b.matmul(b.value, trans_b, g, True, a.shape)
                self._acc(a, ga)
            if b.needs_grad:
                if not trans_b:
                    gb = self.b.matmul(a.value, not trans_a, g, False, b.shape)
                else:
                    gb = self.b.matmul(g, True, a.value, trans_a, b.shape)
                self._acc(b, gb)
        return self._out(y, (m, n), [a, b], back)

    @_op
    def batch_matmul(self, a, b, trans_a=False, trans_b=False):
        """gpu_ops/BatchMatrixMult.py:49-75 (compute), :77 (gradient: the four transpose cases)."""
        lead = a.shape[:-2]
        m = a.shape[-1] if trans_a else a.shape[-2]
        n = b.shape[-2] if trans_b else b.shape[-1]
        ys = tuple(lead) + (m, n)
        y = self.b.batch_matmul(a.value, trans_a, b.value, trans_b, ys)

        def back(g):
            if a.needs_grad:
                if not trans_a:
                    ga = self.b.batch_matmul(g, False, b.value, not trans_b, a.shape)
                else:
                    ga = self.b.batch_matmul(b.value, trans_b, g, True, a.shape)
                self._acc(a, ga)
            if b.needs_grad:
                if not trans_b:
                    gb = self.b.batch_matmul(a.value, not trans_a, g, False, b.shape)
                else:
                    gb = self.b.batch_matmul(g, True, a.value, trans_a, b.shape)
                self._acc(b, gb)
        return self._out(y, ys, [a, b], back)

    @_op
    def add_bias(self, x, bias):
        """x [rows, cols] + broadcast(bias [cols]) (gpu_ops/Broadcast.py:45-59, gradient :65 =
        reduce_sum_axis_zero)."""
        def fwd():
            return self.b.add(x.value, self.b.broadcast_to(bias.value, x.shape), x.shape)

        def back(g):
            self._acc(x, g)
            if bias.needs_grad:
                self._acc(bias, self.b.reduce_sum_axis_zero(g, bias.shape))
        return self._out(fwd(), x.shape, [x, bias], back, saved=[], redo=fwd)

    @_op
    def broadcast_like(self, x, shape):
        """gpu_ops/BroadcastTF.py:46-58 (numpy alignment from the right); gradient = reduce_sum
        over the broadcast axes (gpu_ops/BroadcastShape.py:61)."""
        shape = tuple(shape)

        def fwd():
            return self.b.broadcast_shape(x.value, shape)
        y = fwd()
        diff = len(shape) - len(x.shape)
        axes = [d for d in range(len(shape)) if d < diff or (x.shape[d - diff] == 1 and shape[d] != 1)]

        def back(g):
            if axes:
                self._acc(x, self.b.reduce_sum(g, axes, x.shape))
            else:
                self._acc(x, g)
        return self._out(y, shape, [x], back, saved=[], redo=fwd)

    @_op
    def transpose(self, x, perm):
        """gpu_ops/Transpose.py:44-58 (compute), :60 (gradient: the inverse permutation)."""
        perm = list(perm)
        ys = tuple(x.shape[p] for p in perm)
        def fwd():
            return self.b.transpose(x.value, perm, ys)
        inv = [0] * len(perm)
        for i, p in enumerate(perm):
            inv[p] = i
        return self._out(fwd(), ys, [x], lambda g: self._acc(x, self.b.transpose(g, inv, x.shape)), saved=[], redo=fwd)

    @_op
    def where(self, cond, a, b):
        """gpu_ops/Where.py:41-48 (compute), :50-55 (gradient: where(cond, g, 0) and where(cond, 0, g))."""
        def fwd():
            return self.b.where(cond.value, a.value, b.value, a.shape)
        y = fwd()

        def back(g):
            z = self.b.zeros(a.shape)
            if a.needs_grad:
                self._acc(a, self.b.where(cond.value, g, z, a.shape))
            if b.needs_grad:
                self._acc(b, self.b.where(cond.value, z, g, a.shape))
        return self._out(y, a.shape, [cond, a, b], back, saved=[cond], redo=fwd)

    @_op
    def one_hot(self, ids, classes):
        """gpu_ops/OneHot.py:44-46; no gradient."""
        ys = tuple(ids.shape) + (classes,)
        return self._out(self.b.one_hot(ids.value, ys), ys, [ids], None, saved=[])

    @_op
    def embedding(self, table, ids):
        """gpu_ops/EmbeddingLookUp.py:41-42, gradient :48-49."""
        ys = tuple(ids.shape) + (table.shape[1],)
        y = self.b.embedding(table.value, ids.value, ys)
        return self._out(y, ys, [table, ids], lambda g: self._acc(table, self.b.embedding_grad(g, ids.value, table.shape)),
                         saved=[ids])

    @_op
    def softmax_ce(self, logits, labels, weight=1.0):
        """gpu_ops/SoftmaxCrossEntropy.py:46-67 (compute), :73 and :134-135 (gradient) with an adjoint of one.
        `weight` scales the loss and, through the gradient operator's adjoint argument, its gradient: the
        share of a batch micro-tensor in the mean over the whole batch."""
        assert len(logits.shape) == 2
        loss = self.b.softmax_ce(logits.value, labels.value)
        if weight != 1.0:
            loss = self.b.mul_const(loss, weight, (1,))

        def back(g):
            if weight != 1.0:
                self._acc(logits, self.b.softmax_ce_grad(logits.value, labels.value, logits.shape, weight))
            else:
                self._acc(logits, self.b.softmax_ce_grad(logits.value, labels.value, logits.shape))
        return self._out(loss, (1,), [logits, labels], back, saved=[logits, labels])

    # ---- reverse sweep
    def backward(self, loss):
        """Runs the recorded backward operators in reverse order; the loss adjoint is one
        (gpu_ops/executor.py:175), folded into softmax_ce's gradient."""
        if loss.grad is None:
            loss.grad = True
        for node in reversed(self._nodes):
            v = node.out
            self._before_backward(node)
            if node.back is not None and v.grad is not None:
                node.back(v.grad)
                if v is not loss:
                    v.grad = None      # interior gradients are dropped as soon as they are consumed
            self._after_backward(node)
        self._nodes = []


# ---------------------------------------------------------------- batch micro-tensors on the tape
class _ShapeOnly(object):
    """Backend that computes nothing: every primitive returns None."""

    def __getattr__(self, name):
        return lambda *a, **k: None


def trace(build, inputs, binder_for, fuse_bn_relu=False):
    """Runs `build(tape, binder, cache)` on shapes only and returns the operator calls it makes, in
    order: a list of (method name, args, kwargs), Var arguments being the Vars of that run.
    inputs: name -> shape; binder_for(tape) -> a binder whose parameters need no values."""
    t = Tape(_ShapeOnly())
    t.fuse_bn_relu = fuse_bn_relu
    t._log = []
    cache = {k: t.const(None, shape) for k, shape in inputs.items()}
    build(t, binder_for(t), cache)
    return t._log


# operators whose result for one sample depends on the other samples of the batch: a graph that
# contains one cannot run that part per micro-tensor
COUPLES_SAMPLES = frozenset(["batch_norm", "batch_norm_relu"])


class _PieceTape(Tape):
    """The tape one micro-tensor of a put-off stretch runs on.  It drops a value once its last reader has
    run (`drop_after_forward[t]`: values read by no backward operator whose last forward reader is operator
    t; `drop_after_backward[j]`: values whose last backward reader is operator j) and tells its owner after
    every operator."""

    def __init__(self, backend, owner, drop_after_forward=None, drop_after_backward=None):
        Tape.__init__(self, backend)
        self._owner = owner
        self._drop_f, self._drop_b = drop_after_forward or {}, drop_after_backward or {}

    def _after_forward(self, node):
        for m in self._drop_f.get(node.index, ()):
            self._nodes[m].out.value = None
        self._owner._inside_piece()

    def _after_backward(self, node):
        for m in self._drop_b.get(node.index, ()):
            self._nodes[m].out.value = None
        self._owner._inside_piece()


def _last_readers(nodes):
    """For the operators of one tape: -> (drop_after_forward, drop_after_backward) as _PieceTape takes them.
    The last operator's output (the loss) is never dropped."""
    n = len(nodes)
    last_fwd, need = list(range(n)), [[] for _ in range(n)]
    for t, node in enumerate(nodes):
        for v in node.inputs:
            if v.node >= 0:
                last_fwd[v.node] = max(last_fwd[v.node], t)
        if node.back is not None:
            for v in node.saved:
                if v.node >= 0:
                    need[v.node].append(t)
    drop_f, drop_b = {}, {}
    for m in range(n - 1):
        if need[m]:
            drop_b.setdefault(min(need[m]), []).append(m)
        else:
            drop_f.setdefault(last_fwd[m], []).append(m)
    return drop_f, drop_b


class MicroTape(Tape):
    """A Tape that runs the END of a graph per batch micro-tensor, as TSplit's executor runs a split
    operator as micro-operators on the micro-tensors of its operands (the primitives are
    DLArraySliceForMicroTensor, src/common/c_runtime_api.cc:212-271, and split_shape,
    python/athena/ndarray.py:390-409).

    Operator calls number `split_from` and later are put off while the builder runs: they return Vars
    that carry shapes only.  When call number `total_calls - 1` (the loss) arrives, the stretch runs
    `pieces` times, once per micro-tensor, depth first: for piece i every put-off call is made again
    on a plain tape with the arguments of `piece_calls` (the same builder traced at batch / pieces:
    shapes, permutations and constants of that batch size) and with values of that piece: results of
    the stretch's own earlier calls, or, for a value from outside the stretch, micro-tensor view i of
    it when the trace shows that its shape follows the batch, the whole value when it does not
    (parameters, tables).  Forward and backward of a piece run back to back, so the stretch's
    activations and their gradients exist for one micro-tensor at a time; the loss of piece i is
    weighted with 1 / pieces (equal pieces: the mean over the batch is the mean of the pieces' means).
    The gradients leave the stretch as whole arrays: of a value that follows the batch, written piece
    by piece through micro-tensor views of one array; of a parameter, accumulated over the pieces.
    On the outer tape the stretch is ONE operator whose output is the loss and whose backward
    operators have already run.  Nothing in the stretch may couple the samples of a batch
    (COUPLES_SAMPLES); the batch must divide by `pieces`."""

    def __init__(self, backend, split_from=None, pieces=1, piece_calls=None, total_calls=None):
        Tape.__init__(self, backend)
        self.split_from, self.pieces, self.piece_calls, self.total_calls = split_from, pieces, piece_calls, total_calls
        self._ncalls = 0
        self._put_off = []        # (name, args, kwargs, out Var) of the calls put off so far
        self._deferring = False
        if split_from is not None:
            assert pieces >= 1 and piece_calls is not None and total_calls == len(piece_calls)
            bad = [c[0] for c in piece_calls[split_from:] if c[0] in COUPLES_SAMPLES]
            assert not bad, "operators that couple the samples of a batch cannot run per micro-tensor: %s" % bad[:3]

    def _inside_piece(self):
        pass

    def _call(self, fn, args, kwargs):
        c = self._ncalls
        self._ncalls += 1
        if self.split_from is None or c < self.split_from:
            return Tape._call(self, fn, args, kwargs)
        # put off: the call runs on shapes only and leaves no node
        real, self.b, self._deferring = self.b, _ShapeOnly(), True
        try:
            out = fn(self, *args, **kwargs)
        finally:
            self.b, self._deferring = real, False
        self._put_off.append((fn.__name__, args, kwargs, out))
        if c == self.total_calls - 1:
            return self._run_pieces(out)
        return out

    def _out(self, value, shape, inputs, backward, saved=None, redo=None):
        if self._deferring:
            v = Var(None, shape, any(i.needs_grad for i in inputs))
            v.node = -2          # neither a leaf nor an operator of this tape
            return v
        return Tape._out(self, value, shape, inputs, backward, saved, redo)

    def _readers_of_the_stretch(self, inner_ids):
        """Runs the stretch once on shapes only (the traced calls, stand-ins for the outside values) to learn
        which operator reads each of its values last."""
        dry = Tape(_ShapeOnly())
        env, standin = {}, {}

        def arg_for(actual, traced):
            if not isinstance(actual, Var):
                return traced
            if id(actual) in inner_ids:
                return env[inner_ids[id(actual)]]
            if id(actual) not in standin:
                standin[id(actual)] = Var(None, traced.shape, actual.needs_grad)
            return standin[id(actual)]
        for n, (name, args, kwargs, _) in enumerate(self._put_off):
            _, t_args, t_kwargs = self.piece_calls[self.split_from + n]
            env[n] = getattr(dry, name)(*[arg_for(a, ta) for a, ta in zip(args, t_args)],
                                        **{key: arg_for(kwargs[key], t_kwargs[key]) for key in kwargs})
        return _last_readers(dry._nodes)

    def _run_pieces(self, loss_var):
        k, b = self.pieces, self.b
        inner_ids = {id(c[3]): n for n, c in enumerate(self._put_off)}
        drop_f, drop_b = self._readers_of_the_stretch(inner_ids)
        outside, outside_vars = {}, []          # id(Var) -> [Var, follows the batch, whole gradient array or None]
        total = None
        for i in range(k):
            piece_tape = _PieceTape(b, self, drop_f, drop_b)
            env = {}                            # put-off call -> its result for this piece
            wrapped = {}                        # id(outside Var) -> its Var on the piece's tape

            def arg_for(actual, traced):
                if not isinstance(actual, Var):
                    return traced               # shapes, permutations, constants: those of the piece's batch size
                if id(actual) in inner_ids:
                    return env[inner_ids[id(actual)]]
                if id(actual) not in wrapped:
                    follows = tuple(traced.shape) != tuple(actual.shape)
                    if follows:
                        assert tuple(traced.shape[1:]) == tuple(actual.shape[1:]) and traced.shape[0] * k == actual.shape[0], \
                            (actual.shape, traced.shape, k)
                    if id(actual) not in outside:
                        outside[id(actual)] = [actual, follows, None]
                        outside_vars.append(actual)
                    value = b.piece(actual.value, k, i) if follows else actual.value
                    wrapped[id(actual)] = Var(value, traced.shape, actual.needs_grad, actual.name)
                return wrapped[id(actual)]

            for n, (name, args, kwargs, _) in enumerate(self._put_off):
                t_name, t_args, t_kwargs = self.piece_calls[self.split_from + n]
                assert t_name == name and len(t_args) == len(args), "the graph differs from the traced one"
                p_args = [arg_for(a, ta) for a, ta in zip(args, t_args)]
                p_kwargs = {key: arg_for(kwargs[key], t_kwargs[key]) for key in kwargs}
                if n == len(self._put_off) - 1:
                    assert name == "softmax_ce", "a stretch run per micro-tensor ends with the loss"
                    p_kwargs["weight"] = 1.0 / k
                env[n] = getattr(piece_tape, name)(*p_args, **p_kwargs)
            piece_loss = env[len(self._put_off) - 1]
            total = piece_loss.value if total is None else b.add(total, piece_loss.value, (1,))
            piece_tape.backward(piece_loss)
            for key, w in wrapped.items():
                actual, follows, whole = outside[key]
                if not actual.needs_grad or w.grad is None:
                    continue
                if follows:
                    if whole is None:
                        whole = outside[key][2] = b.empty(actual.shape)
                    b.assign(b.piece(whole, k, i), w.grad)
                else:
                    self._acc(actual, w.grad)           # a parameter: summed over the pieces
                w.grad = None
            del piece_tape, env, wrapped, piece_loss
        for v in outside_vars:
            whole = outside[id(v)][2]
            if whole is not None:
                self._acc(v, whole)
        self._put_off = []
        # on this tape the stretch is one operator: it read the outside values, its output is the loss
        # and its backward operators have run
        out = Tape._out(self, total, (1,), outside_vars, None, saved=[])
        out.needs_grad = False
        return out
