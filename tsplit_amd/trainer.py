"""Minimal executor for sequential conv nets, driving the operator library through
`gpu_links` exactly as the reference's executor loop drives it.

Reproduces, for a layer list, what the reference does for a graph: one NDArray per node
output (python/athena/gpu_ops/executor.py:71-92), a forward sweep that calls each op's GPU
symbol on one compute stream (executor.py:140-152), the backward nodes its autodiff creates
(conv -> gradient_of_filter + gradient_of_data, matmul -> two transposed matmuls, relu ->
relu_gradient, maxpool -> max_pooling2d_gradient, softmaxCE -> its gradient seeded with ones:
executor.py:160-196), filter gradients issued before data gradients (executor.py:327-332),
the data gradient of the first layer never evaluated, then one optimizer call per parameter
(python/athena/optimizer.py:95-176).

The TSplit part: `split={layer_index: pieces}` runs that conv layer (forward, both
backward passes) on `pieces` zero-copy batch micro-tensors (DLArraySliceForMicroTensor);
per-piece filter gradients are summed with DLGpuMatrixElementwiseAdd.  BatchNorm always
sees the whole batch: its statistics are batch statistics, so a BN over a micro-batch is
a different function.

Layer spec entries:
    ("conv", name, Cin, Cout, k, pad, stride) | ("bn", name, C) | ("relu",) |
    ("maxpool", k, pad, stride) | ("flatten",) | ("fc", name, n_in, n_out)
"""
import numpy as np

from . import gpu_links as L
from . import ndarray
from .stream import create_stream_handle


def mlp_spec(sizes=(784, 256, 256, 10)):
    """784 -> 256 -> 256 -> 10 without biases, Relu between layers."""
    spec = []
    for i in range(len(sizes) - 1):
        spec.append(("fc", "mlp_fc%d" % (i + 1), sizes[i], sizes[i + 1]))
        if i < len(sizes) - 2:
            spec.append(("relu",))
    return spec


def vgg16_spec(num_classes=1000, in_hw=224, fc_width=4096):
    return vgg_spec(16, num_classes, in_hw, fc_width)


def vgg19_spec(num_classes=1000, in_hw=224):
    return vgg_spec(19, num_classes, in_hw)


def vgg_spec(depth=16, num_classes=1000, in_hw=224, fc_width=4096):
    """VGG-16 / VGG-19 as examples/imagenet_vgg.py:24-98 builds them: 13 or 16 x (conv3x3 pad 1, BN,
    Relu), 5 max-pools 2x2/2, flatten, three bias-free fully connected layers with no activation
    in between (`fc_width` units in the two hidden ones: 4096 in the example)."""
    per_block = {16: (2, 2, 3, 3, 3), 19: (2, 2, 4, 4, 4)}[depth]
    spec = []
    cin = 3
    for bi, (n, cout) in enumerate(zip(per_block, (64, 128, 256, 512, 512)), 1):
        for li in range(1, n + 1):
            name = "vgg_block%d_layer%d" % (bi, li)
            spec += [("conv", name, cin, cout, 3, 1, 1), ("bn", name + "_bn", cout), ("relu",)]
            cin = cout
        spec.append(("maxpool", 2, 0, 2))
    spec.append(("flatten",))
    feat = 512 * (in_hw // 32) ** 2
    spec += [("fc", "vgg_fc1", feat, fc_width), ("fc", "vgg_fc2", fc_width, fc_width), ("fc", "vgg_fc3", fc_width, num_classes)]
    return spec


def param_shapes(spec):
    shapes = {}
    for layer in spec:
        if layer[0] == "conv":
            _, name, cin, cout, k, _, _ = layer
            shapes[name + "_weight"] = (cout, cin, k, k)
        elif layer[0] in ("bn", "bnrelu", "bnrelupool"):
            _, name, c = layer
            shapes[name + "_scale"] = (1, c, 1, 1)
            shapes[name + "_bias"] = (1, c, 1, 1)
        elif layer[0] == "fc":
            _, name, n_in, n_out = layer
            shapes[name + "_weight"] = (n_in, n_out)
    return shapes


def init_params(spec, seed=123, scheme="he"):
    """Seeded host-side initialisation.  "he": N(0, sqrt(2/fan_in)) weights, BN scale 1, bias 0.
    "normal0.1": N(0, 0.1) everywhere (what examples/imagenet_vgg.py:14-21 draws)."""
    rng = np.random.RandomState(seed)
    params = {}
    for name, shape in param_shapes(spec).items():
        if scheme == "normal0.1":
            params[name] = rng.normal(scale=0.1, size=shape).astype(np.float32)
        elif name.endswith("_scale"):
            params[name] = np.ones(shape, np.float32)
        elif name.endswith("_bias"):
            params[name] = np.zeros(shape, np.float32)
        else:
            fan_in = int(np.prod(shape[1:])) if len(shape) == 4 else shape[0]
            params[name] = rng.normal(scale=np.sqrt(2.0 / fan_in), size=shape).astype(np.float32)
    return params


def _out_shape(layer, s):
    kind = layer[0]
    if kind == "conv":
        _, _, _, cout, k, pad, stride = layer
        return (s[0], cout, (s[2] + 2 * pad - k) // stride + 1, (s[3] + 2 * pad - k) // stride + 1)
    if kind in ("bn", "relu", "bnrelu"):
        return s
    if kind == "bnrelupool":       # BatchNorm + Relu + 2x2 / stride 2 max pooling as one layer
        return (s[0], s[1], s[2] // 2, s[3] // 2)
    if kind == "maxpool":
        _, k, pad, stride = layer
        return (s[0], s[1], (s[2] + 2 * pad - k) // stride + 1, (s[3] + 2 * pad - k) // stride + 1)
    if kind == "flatten":
        return (s[0], int(np.prod(s[1:])))
    if kind == "fc":
        return (s[0], layer[3])
    raise ValueError(kind)


class Trainer(object):
    def __init__(self, spec, params, input_shape, num_classes, ctx=None, optimizer=("sgd", 0.1),
                 split=None, bn_eps=0.01, timer=None, fuse_bn_relu=False, conv_bn_stats=False,
                 multi_tensor_update=False, fuse_max_pool=False):
        self.spec = list(spec)
        # with fuse_bn_relu a ("bn", ...) layer directly followed by ("relu",) runs as ONE fused call
        # in each direction (symbols outside the reference's ABI); the Relu layer's own arrays are
        # then never touched: the fused output and input gradient live in the BN layer's slots
        self.fused = set()
        if fuse_bn_relu:
            self.fused = {li for li, l in enumerate(self.spec[:-1]) if l[0] == "bn" and self.spec[li + 1][0] == "relu"}
        # with fuse_max_pool a fused pair directly followed by ("maxpool", 2, 0, 2) on planes of even height and
        # width runs as ONE call each way together with the pooling (symbols outside the reference's ABI): the
        # activation in front of the pooling is never written (filled in below, where the shapes are known)
        self.fused_pool = set()
        want_pool = bool(fuse_max_pool and fuse_bn_relu)
        # with conv_bn_stats a ("conv", ...) layer directly followed by ("bn", ...) hands the BatchNorm its
        # batch statistics (one row of sums per micro-tensor; symbols outside the reference's ABI), so
        # the BatchNorm reads the convolution's output once instead of twice
        self.stats_of = {}
        if conv_bn_stats:
            self.stats_of = {li: None for li, l in enumerate(self.spec[:-1])
                             if l[0] == "conv" and self.spec[li + 1][0] == "bn"}
        # with multi_tensor_update the optimizer updates every parameter in ONE launch (a symbol outside
        # the reference's ABI) instead of one call per parameter
        self.multi_tensor_update = multi_tensor_update
        # optional per-call timing hook: timer.begin(stream) / timer.end(stream, tag, work, unit)
        self.timer = timer
        self.ctx = ctx if ctx is not None else ndarray.gpu(0)
        self.stream = create_stream_handle(self.ctx)
        self.optimizer = optimizer
        self.split = dict(split or {})
        self.eps = bn_eps
        self.params = {k: ndarray.array(v, self.ctx) for k, v in params.items()}
        self.grads = {k: ndarray.empty(v.shape, self.ctx) for k, v in params.items()}
        self.state = {}
        if optimizer[0] == "momentum":
            self.state = {k: ndarray.array(np.zeros(v.shape, np.float32), self.ctx) for k, v in params.items()}
        # one array per node output, one per node gradient
        self.acts = [None]          # acts[0] is the input, bound per step
        self.dacts = [None]
        self.saved = {}
        self.dw_piece = {}
        s = tuple(input_shape)
        self.shapes = [s]
        for li, layer in enumerate(self.spec):
            if (want_pool and li in self.fused and li + 2 < len(self.spec) and tuple(self.spec[li + 2]) == ("maxpool", 2, 0, 2)
                    and s[2] % 2 == 0 and s[3] % 2 == 0):
                self.fused_pool.add(li)
            s = _out_shape(layer, s)
            self.shapes.append(s)
            # the BN output of a fused pair never exists, nor the Relu output in front of a fused pooling
            unused = li in self.fused or (layer[0] == "relu" and li - 1 in self.fused_pool)
            self.acts.append(None if unused else ndarray.empty(s, self.ctx))
            self.dacts.append(None if unused else ndarray.empty(s, self.ctx))
            if layer[0] == "bn":
                c = layer[2]
                self.saved[li] = (ndarray.empty((1, c, 1, 1), self.ctx), ndarray.empty((1, c, 1, 1), self.ctx))
            if layer[0] == "conv" and li in self.split:
                self.acts[-1].split_tensor(self.split[li])
                self.dacts[-1].split_tensor(self.split[li])
                # per-piece filter gradient, summed into the layer's gradient
                self.dw_piece[li] = ndarray.empty(param_shapes([layer])[layer[1] + "_weight"], self.ctx)
            if li in self.stats_of:
                # [pieces][Cout][2] doubles in float32 storage
                self.stats_of[li] = ndarray.empty((self.split.get(li, 1) * layer[3] * 4,), self.ctx)
        assert self.shapes[-1] == (input_shape[0], num_classes), (self.shapes[-1], num_classes)
        self.loss = ndarray.empty((1,), self.ctx)
        self.ones = ndarray.empty((1,), self.ctx)
        L.array_set(self.ones, 1.0, self.stream)          # adjoint seed (executor.py:175)
        for li in self.split:
            if li > 0:
                self.acts[li].split_tensor(self.split[li])
                self.dacts[li].split_tensor(self.split[li])

    def _run(self, tag, work, unit, fn, *args, moved=None):
        """Issue one operator call on the compute stream; `work` is its algorithmic FLOP or
        byte count (each distinct input read once, each output written once); `moved` gives the
        byte count of a call whose work is counted in FLOP but which sits near the ridge."""
        if self.timer is None:
            fn(*args, self.stream)
        else:
            self.timer.begin(self.stream)
            fn(*args, self.stream)
            self.timer.end(self.stream, tag, work, unit, moved)

    @staticmethod
    def _n(shape):
        return int(np.prod(shape))

    @staticmethod
    def _tile(rows):
        return "64x256" if rows <= 64 else "128x128"

    # ---------------------------------------------------------------- forward
    def forward(self, x, labels):
        n = self._n
        self.acts[0] = x
        if 0 in self.split:
            x.split_tensor(self.split[0])
        for li, layer in enumerate(self.spec):
            a, out = self.acts[li], self.acts[li + 1]
            kind = layer[0]
            if kind == "conv":
                _, name, cin, cout, k, pad, stride = layer
                w = self.params[name + "_weight"]
                thin = cin * k * k <= 32      # a first layer (3 input channels): bound by HBM, timed in bytes
                pairs = list(zip(a.sTensor, out.sTensor)) if li in self.split else [(a, out)]
                xs = pairs[0][0].shape
                wino = L.conv_takes_winograd(xs[0], cin, cout, xs[2], xs[3], k, pad, stride)
                tag = "conv_fwd_thin" if thin else "conv_fwd_winograd" if wino else "conv_fwd_" + self._tile(cout)
                for i, (xa, ya) in enumerate(pairs):
                    if li in self.stats_of:
                        call, args = L.conv2d_batch_norm_stats, (xa, w, ya, self.stats_of[li], i, pad, pad, stride)
                    else:
                        call, args = L.CuDNN_conv2d, (xa, w, ya, pad, pad, stride)
                    if thin:
                        self._run(tag, 4.0 * (n(xa.shape) + n(w.shape) + n(ya.shape)), "byte", call, *args)
                    else:
                        self._run(tag, 2.0 * n(ya.shape) * cin * k * k, "flop", call, *args)
            elif kind == "bn" and li in self.fused_pool:
                name = layer[1]
                sm, sv = self.saved[li]
                pooled = self.acts[li + 3]
                from_stats = li - 1 in self.stats_of
                self._run("bn_relu_pool_fwd_from_stats" if from_stats else "bn_relu_pool_fwd", 4.0 * (n(a.shape) + n(pooled.shape)),
                          "byte", L.batch_norm_relu_max_pool, a, self.params[name + "_scale"], self.params[name + "_bias"],
                          pooled, sm, sv, self.eps, self.stats_of[li - 1] if from_stats else None,
                          self.split.get(li - 1, 1) if from_stats else 0)
            elif kind == "bn" and li - 1 in self.stats_of:
                name = layer[1]
                sm, sv = self.saved[li]
                fused = li in self.fused
                self._run("bn_relu_fwd_from_stats" if fused else "bn_fwd_from_stats", 8.0 * n(a.shape), "byte",
                          L.batch_norm_from_stats, a, self.stats_of[li - 1], self.split.get(li - 1, 1),
                          self.params[name + "_scale"], self.params[name + "_bias"],
                          self.acts[li + 2] if fused else out, sm, sv, self.eps, fused)
            elif kind == "bn" and li in self.fused:
                name = layer[1]
                sm, sv = self.saved[li]
                # writes the Relu layer's output directly
                self._run("bn_relu_fwd", 8.0 * n(a.shape), "byte", L.batch_norm_relu, a, self.params[name + "_scale"],
                          self.params[name + "_bias"], self.acts[li + 2], sm, sv, self.eps)
            elif kind == "bn":
                name = layer[1]
                sm, sv = self.saved[li]
                self._run("bn_fwd", 8.0 * n(a.shape), "byte", L.CuDNN_Batch_Normalization, a,
                          self.params[name + "_scale"], self.params[name + "_bias"], out, sm, sv, 0.99, self.eps)
            elif kind == "relu" and li - 1 in self.fused:
                pass
            elif kind == "relu":
                self._run("relu_fwd", 8.0 * n(a.shape), "byte", L.relu, a, out)
            elif kind == "maxpool" and li - 2 in self.fused_pool:
                pass
            elif kind == "maxpool":
                _, k, pad, stride = layer
                self._run("maxpool_fwd", 4.0 * (n(a.shape) + n(out.shape)), "byte", L.CuDNN_max_pooling2d, a, k, k, out,
                          pad, stride)
            elif kind == "flatten":
                self._run("reshape", 8.0 * n(a.shape), "byte", L.array_reshape, a, out)
            elif kind == "fc":
                _, name, n_in, n_out = layer
                self._run("matmul_" + self._tile(a.shape[0]), 2.0 * a.shape[0] * n_in * n_out, "flop",
                          L.matrix_multiply, a, False, self.params[name + "_weight"], False, out,
                          moved=4.0 * (a.shape[0] * n_in + n_in * n_out + a.shape[0] * n_out))
        self._run("softmax_ce_fwd", 8.0 * n(self.acts[-1].shape), "byte", L.softmax_cross_entropy, self.acts[-1],
                  labels, self.loss)
        return self.loss

    # ---------------------------------------------------------------- backward
    def backward(self, labels):
        n = self._n
        self._run("softmax_ce_bwd", 12.0 * n(self.acts[-1].shape), "byte", L.softmax_cross_entropy_gradient,
                  self.acts[-1], labels, self.ones, self.dacts[-1])
        for li in range(len(self.spec) - 1, -1, -1):
            layer = self.spec[li]
            a, g_out, g_in = self.acts[li], self.dacts[li + 1], self.dacts[li]
            kind = layer[0]
            first = li == 0
            if kind == "conv":
                _, name, cin, cout, k, pad, stride = layer
                w, dw = self.params[name + "_weight"], self.grads[name + "_weight"]
                split = li in self.split
                xs = a.sTensor if split else [a]
                gs = g_out.sTensor if split else [g_out]
                for i, (xa, ga) in enumerate(zip(xs, gs)):
                    # filter gradient first, as the reference reorders it (executor.py:327-332)
                    if cin * k * k <= 32:
                        self._run("conv_bwd_filter_thin", 4.0 * (n(xa.shape) + n(ga.shape) + n(dw.shape)), "byte",
                                  L.CuDNN_conv2d_gradient_of_filter, xa, ga, dw if i == 0 else self.dw_piece[li],
                                  pad, pad, stride)
                    else:
                        wino = L.conv_takes_winograd(xa.shape[0], cin, cout, xa.shape[2], xa.shape[3], k, pad, stride,
                                                     filter_gradient=True)
                        self._run("conv_bwd_filter_winograd" if wino else "conv_bwd_filter_" + self._tile(cout),
                                  2.0 * n(ga.shape) * cin * k * k, "flop",
                                  L.CuDNN_conv2d_gradient_of_filter, xa, ga, dw if i == 0 else self.dw_piece[li],
                                  pad, pad, stride)
                    if i > 0:
                        self._run("add", 12.0 * n(dw.shape), "byte", L.matrix_elementwise_add, dw, self.dw_piece[li], dw)
                if not first:
                    gis = g_in.sTensor if split else [g_in]
                    wino = L.conv_takes_winograd(gis[0].shape[0], cin, cout, gis[0].shape[2], gis[0].shape[3], k, pad, stride,
                                                 data_gradient=True)
                    for ga, gi in zip(gs, gis):
                        self._run("conv_bwd_data_winograd" if wino else "conv_bwd_data_" + self._tile(cin),
                                  2.0 * n(ga.shape) * cin * k * k, "flop",
                                  L.CuDNN_conv2d_gradient_of_data, w, ga, gi, pad, pad, stride)
            elif kind == "bn" and li in self.fused_pool:
                name = layer[1]
                sm, sv = self.saved[li]
                gp = self.dacts[li + 3]      # the gradient behind the pooling
                self._run("bn_relu_pool_bwd", 4.0 * (2 * n(a.shape) + n(gp.shape)), "byte", L.batch_norm_relu_max_pool_gradient,
                          gp, a, self.params[name + "_scale"], self.params[name + "_bias"], g_in,
                          self.grads[name + "_scale"], self.grads[name + "_bias"], sm, sv, self.eps)
            elif kind == "bn" and li in self.fused:
                name = layer[1]
                sm, sv = self.saved[li]
                # consumes the gradient behind the Relu layer
                self._run("bn_relu_bwd", 12.0 * n(a.shape), "byte", L.batch_norm_relu_gradient, self.dacts[li + 2], a,
                          self.params[name + "_scale"], self.params[name + "_bias"], g_in,
                          self.grads[name + "_scale"], self.grads[name + "_bias"], sm, sv, self.eps)
            elif kind == "bn":
                name = layer[1]
                sm, sv = self.saved[li]
                self._run("bn_bwd", 12.0 * n(a.shape), "byte", L.CuDNN_Batch_Normalization_gradient, g_out, a,
                          self.params[name + "_scale"], g_in, self.grads[name + "_scale"],
                          self.grads[name + "_bias"], sm, sv, self.eps)
            elif kind == "relu" and li - 1 in self.fused:
                pass
            elif kind == "relu":
                self._run("relu_bwd", 12.0 * n(a.shape), "byte", L.relu_gradient, a, g_out, g_in)
            elif kind == "maxpool" and li - 2 in self.fused_pool:
                pass
            elif kind == "maxpool":
                _, k, pad, stride = layer
                self._run("maxpool_bwd", 4.0 * (2 * n(a.shape) + n(g_out.shape)), "byte",
                          L.CuDNN_max_pooling2d_gradient, self.acts[li + 1], g_out, a, k, k, g_in, pad, stride)
            elif kind == "flatten":
                self._run("reshape", 8.0 * n(a.shape), "byte", L.array_reshape, g_out, g_in)
            elif kind == "fc":
                _, name, n_in, n_out = layer
                w = self.params[name + "_weight"]
                m = a.shape[0]
                moved = 4.0 * (m * n_in + n_in * n_out + m * n_out)
                self._run("matmul_" + self._tile(n_in), 2.0 * m * n_in * n_out, "flop", L.matrix_multiply, a, True,
                          g_out, False, self.grads[name + "_weight"], moved=moved)
                if not first:
                    self._run("matmul_" + self._tile(m), 2.0 * m * n_in * n_out, "flop", L.matrix_multiply, g_out,
                              False, w, True, g_in, moved=moved)

    # ---------------------------------------------------------------- update
    def update(self):
        if self.multi_tensor_update and self.optimizer[0] in ("sgd", "momentum"):
            names = list(self.params)
            total = sum(self._n(self.params[k].shape) for k in names)
            ps, gs = [self.params[k] for k in names], [self.grads[k] for k in names]
            if self.optimizer[0] == "sgd":
                self._run("sgd_multi", 12.0 * total, "byte", L.optimizer_update_multi, ps, gs, None, self.optimizer[1], 0.0, False)
            else:
                self._run("momentum_multi", 20.0 * total, "byte", L.optimizer_update_multi, ps, gs,
                          [self.state[k] for k in names], self.optimizer[1], self.optimizer[2], False)
            return
        for name, p in self.params.items():
            g = self.grads[name]
            if self.optimizer[0] == "sgd":
                self._run("sgd", 12.0 * self._n(p.shape), "byte", L.sgd_update, p, g, self.optimizer[1])
            elif self.optimizer[0] == "momentum":
                self._run("momentum", 20.0 * self._n(p.shape), "byte", L.momentum_update, p, g, self.state[name],
                          self.optimizer[1], self.optimizer[2], False)
            else:
                raise ValueError(self.optimizer[0])

    def step(self, x, labels):
        """One training step, asynchronous on self.stream; returns the (device) loss array."""
        self.forward(x, labels)
        self.backward(labels)
        self.update()
        return self.loss

    def record_step(self, x, labels):
        """Records one training step on (x, labels) into a graph and returns it: graph.launch(
        self.stream) then runs the whole step with one host call, reading whatever x and labels
        hold at that time.  For nets whose step is bound by the host's launch rate.  The step must
        have run once before (first-use set-up cannot be recorded); per-call timers stay off."""
        from .stream import recording
        timer, self.timer = self.timer, None
        try:
            with recording(self.stream) as rec:
                self.step(x, labels)
        finally:
            self.timer = timer
        return rec.graph

    def sync(self):
        self.stream.sync()

    def loss_value(self):
        self.sync()
        return float(self.loss.asnumpy()[0])
