"""Graph builders of the reference's example networks on the tape of graph.py.

Topologies follow the reference's examples node for node:
  resnet        examples/imagenet_resnet.py:26-122   (bottleneck blocks; the shortcut branch is
                conv + BN + Relu, the Relu precedes the residual add, stride 2 sits on the 3x3)
  inception_v4  examples/imagenet_inceptionv4.py:84-251 ("same" padding = (k - stride) / 2 per
                axis, two-input channel concats chained, 3x3 average pools with padding 1)
  transformer   examples/transformer.py:56-287 (dense = matmul + broadcast bias; attention
                scores are masked and used without a softmax, layer norm and dropout are
                commented out there and absent here; logits reuse the embedding table)
Every size is an argument so that the tests can run the same graphs small enough for the
numpy backend; the defaults are the sizes of the reference's benchmark configurations.
Parameters are created on first use by name from one seeded generator (ParamStore), so two
tapes (device and numpy) built from one store see identical values.
"""
import collections

import numpy as np


class ParamStore(object):
    """name -> float32 numpy array, created on first request in request order."""

    def __init__(self, seed=123):
        self.rng = np.random.RandomState(seed)
        self.values = collections.OrderedDict()
        self.trainable = {}

    def get(self, name, shape, init, trainable=True):
        if name not in self.values:
            shape = tuple(int(s) for s in shape)
            if callable(init):
                v = init(shape)
            elif init == "he":          # conv OIHW or fc [in, out]
                fan_in = int(np.prod(shape[1:])) if len(shape) == 4 else shape[0]
                v = self.rng.normal(0.0, np.sqrt(2.0 / fan_in), size=shape)
            elif init == "one":
                v = np.ones(shape)
            elif init == "zero":
                v = np.zeros(shape)
            else:                        # a standard deviation
                v = self.rng.normal(0.0, float(init), size=shape)
            self.values[name] = np.ascontiguousarray(v, dtype=np.float32)
            self.trainable[name] = trainable
        assert self.values[name].shape == tuple(shape), (name, self.values[name].shape, shape)
        return self.values[name]


class Binder(object):
    """Binds a ParamStore to one tape: one Var per name (shared parameters accumulate)."""

    def __init__(self, tape, store):
        self.t, self.store, self.vars = tape, store, collections.OrderedDict()
        self._n = 0
        self._consts = {}

    def unique(self, prefix):
        self._n += 1
        return "%s%d" % (prefix, self._n)

    def get(self, name, shape, init, trainable=True):
        if name not in self.vars:
            v = self.store.get(name, shape, init, trainable)
            mk = self.t.param if trainable else self.t.const
            self.vars[name] = mk(self.t.b.from_numpy(v), v.shape, name)
        return self.vars[name]

    def input(self, array):
        a = np.ascontiguousarray(array, dtype=np.float32)
        return self.t.const(self.t.b.from_numpy(a), a.shape)

    def constant(self, key, make):
        """A constant tensor built and uploaded once per binder: make() -> numpy array."""
        if key not in self._consts:
            a = np.ascontiguousarray(make(), dtype=np.float32)
            self._consts[key] = (self.t.b.from_numpy(a), a.shape)
        value, shape = self._consts[key]
        return self.t.const(value, shape)

    def grads(self):
        """name -> numpy gradient of every trainable parameter that received one."""
        return collections.OrderedDict((k, self.t.b.to_numpy(v.grad)) for k, v in self.vars.items()
                                       if v.needs_grad and v.grad is not None)

    def sgd_step(self, lr):
        """In-place SGD on the bound parameters; the store keeps the host copies in step."""
        for k, v in self.vars.items():
            if v.needs_grad and v.grad is not None:
                self.t.b.sgd(v.value, v.grad, lr)
                v.grad = None

    def pull(self):
        for k, v in self.vars.items():
            if v.needs_grad:
                self.store.values[k] = np.ascontiguousarray(self.t.b.to_numpy(v.value), dtype=np.float32).reshape(v.shape)


class ShapeBinder(Binder):
    """A Binder for runs that only need shapes (recording a graph, counting bytes): a constant's array is
    built once per process to learn its shape and never again."""
    _shapes = {}

    def constant(self, key, make):
        if key not in ShapeBinder._shapes:
            ShapeBinder._shapes[key] = tuple(np.shape(make()))
        shape = ShapeBinder._shapes[key]
        if key not in self._consts:
            self._consts[key] = (self.t.b.from_numpy(np.broadcast_to(np.float32(0), shape)), shape)
        value, shape = self._consts[key]
        return self.t.const(value, shape)


# ------------------------------------------------------------------ ResNet (bottleneck)
def _bn_relu(t, b, x, name, eps):
    c = x.shape[1]
    return t.bn_then_relu(x, b.get(name + "_scale", (1, c, 1, 1), "one"), b.get(name + "_bias", (1, c, 1, 1), "zero"), eps)


def _conv(t, b, x, cout, k, stride, pad, name):
    w = b.get(name + "_weight", (cout, x.shape[1], k, k), "he")
    return t.conv2d(x, w, pad, pad, stride)


def _bottleneck_stage(t, b, x, cout, num_blocks, first, name, eps):
    """examples/imagenet_resnet.py:46-81."""
    s = 1 if first else 2
    mid = cout // 4
    identity = _bn_relu(t, b, _conv(t, b, x, cout, 1, s, 0, name + "_conv0"), name + "_bn0", eps)
    x = _bn_relu(t, b, _conv(t, b, x, mid, 1, 1, 0, name + "_conv1"), name + "_bn1", eps)
    x = _bn_relu(t, b, _conv(t, b, x, mid, 3, s, 1, name + "_conv2"), name + "_bn2", eps)
    x = _bn_relu(t, b, _conv(t, b, x, cout, 1, 1, 0, name + "_conv3"), name + "_bn3", eps)
    x = t.add(x, identity)
    for i in range(1, num_blocks):
        identity = x
        x = _bn_relu(t, b, _conv(t, b, x, mid, 1, 1, 0, name + "_conv%d" % (3 * i + 1)), name + "_bn%d" % (3 * i + 1), eps)
        x = _bn_relu(t, b, _conv(t, b, x, mid, 3, 1, 1, name + "_conv%d" % (3 * i + 2)), name + "_bn%d" % (3 * i + 2), eps)
        x = _bn_relu(t, b, _conv(t, b, x, cout, 1, 1, 0, name + "_conv%d" % (3 * i + 3)), name + "_bn%d" % (3 * i + 3), eps)
        x = t.add(x, identity)
    return x


def resnet(t, b, x, labels, blocks=(3, 4, 6, 3), base=64, classes=1000, eps=0.01):
    """ResNet-50 by default (examples/imagenet_resnet.py:88-122).  x: Var [N,3,H,W]; labels:
    Var [N,classes] one-hot.  The closing average pool spans the whole final plane (7x7 at
    224x224 as in the reference).  Returns (loss, logits)."""
    x = _bn_relu(t, b, _conv(t, b, x, base, 7, 2, 3, "resnet_initial_conv"), "resnet_initial_bn", eps)
    x = t.max_pool(x, 3, 1, 2)
    width = 4 * base
    for i, n in enumerate(blocks):
        x = _bottleneck_stage(t, b, x, width, n, i == 0, "resnet_block%d" % (i + 1), eps)
        width *= 2
    assert x.shape[2] == x.shape[3]
    x = t.avg_pool(x, x.shape[2], 0, x.shape[2])
    x = t.reshape(x, (x.shape[0], -1))
    logits = t.matmul(x, b.get("resnet_final_fc_weight", (x.shape[1], classes), "he"))
    return t.softmax_ce(logits, labels), logits


# ------------------------------------------------------------------ Inception-v4
def _conv_bn(t, b, x, cout, kh, kw, stride=1, same=True, eps=0.01):
    """examples/imagenet_inceptionv4.py:84-95."""
    name = b.unique("inc")
    w = b.get(name + "_W", (cout, x.shape[1], kh, kw), "he")
    ph, pw = ((kh - stride) // 2, (kw - stride) // 2) if same else (0, 0)
    x = t.conv2d(x, w, ph, pw, stride)
    return t.bn_then_relu(x, b.get(name + "_scale", (1, cout, 1, 1), "one"), b.get(name + "_bias", (1, cout, 1, 1), "zero"), eps)


def _cat(t, parts):
    x = parts[0]
    for p in parts[1:]:
        x = t.concat(x, p, 1)
    return x


def inception_v4(t, b, x, labels, n_a=4, n_b=7, n_c=3, div=1, classes=1000, eps=0.01):
    """examples/imagenet_inceptionv4.py:97-251.  `div` divides every channel width (1 = the
    reference's widths); the closing average pool spans the final plane (8x8 at 299x299)."""
    def c(n):
        return max(1, n // div)

    def cb(x, cout, kh, kw, stride=1, same=True):
        return _conv_bn(t, b, x, c(cout), kh, kw, stride, same, eps)

    # stem (:189-213)
    net = cb(x, 32, 3, 3, 2, False)
    net = cb(net, 32, 3, 3, 1, False)
    net = cb(net, 64, 3, 3)
    net = _cat(t, [t.max_pool(net, 3, 0, 2), cb(net, 96, 3, 3, 2, False)])
    b0 = cb(cb(net, 64, 1, 1), 96, 3, 3, 1, False)
    b1 = cb(cb(cb(cb(net, 64, 1, 1), 64, 1, 7), 64, 7, 1), 96, 3, 3, 1, False)
    net = _cat(t, [b0, b1])
    net = _cat(t, [cb(net, 192, 3, 3, 2, False), t.max_pool(net, 3, 0, 2)])
    for _ in range(n_a):                                   # :97-114
        b0 = cb(net, 96, 1, 1)
        b1 = cb(cb(net, 64, 1, 1), 96, 3, 3)
        b2 = cb(cb(cb(net, 64, 1, 1), 96, 3, 3), 96, 3, 3)
        b3 = cb(t.avg_pool(net, 3, 1, 1), 96, 1, 1)
        net = _cat(t, [b0, b1, b2, b3])
    b0 = cb(net, 384, 3, 3, 2, False)                       # reduction A :116-127
    b1 = cb(cb(cb(net, 192, 1, 1), 224, 3, 3), 256, 3, 3, 2, False)
    net = _cat(t, [b0, b1, t.max_pool(net, 3, 0, 2)])
    for _ in range(n_b):                                   # :129-150
        b0 = cb(net, 384, 1, 1)
        b1 = cb(cb(cb(net, 192, 1, 1), 224, 1, 7), 256, 7, 1)
        b2 = cb(cb(cb(cb(cb(net, 192, 1, 1), 192, 7, 1), 224, 1, 7), 224, 7, 1), 256, 1, 7)
        b3 = cb(t.avg_pool(net, 3, 1, 1), 128, 1, 1)
        net = _cat(t, [b0, b1, b2, b3])
    b0 = cb(cb(net, 192, 1, 1), 192, 3, 3, 2, False)        # reduction B :152-165
    b1 = cb(cb(cb(cb(net, 256, 1, 1), 256, 1, 7), 320, 7, 1), 320, 3, 3, 2, False)
    net = _cat(t, [b0, b1, t.max_pool(net, 3, 0, 2)])
    for _ in range(n_c):                                   # :167-187
        b0 = cb(net, 256, 1, 1)
        b1 = cb(net, 384, 1, 1)
        b1 = _cat(t, [cb(b1, 256, 1, 3), cb(b1, 256, 3, 1)])
        b2 = cb(cb(cb(net, 384, 1, 1), 448, 3, 1), 512, 1, 3)
        b2 = _cat(t, [cb(b2, 256, 1, 3), cb(b2, 256, 3, 1)])
        b3 = cb(t.avg_pool(net, 3, 1, 1), 256, 1, 1)
        net = _cat(t, [b0, b1, b2, b3])
    assert net.shape[2] == net.shape[3]
    net = t.avg_pool(net, net.shape[2], 0, 1)               # :250-253
    net = t.reshape(net, (net.shape[0], -1))
    logits = t.matmul(net, b.get("inc_fc_W", (net.shape[1], classes), "he"))
    logits = t.add_bias(logits, b.get("inc_fc_b", (classes,), "zero"))
    return t.softmax_ce(logits, labels), logits


# ------------------------------------------------------------------ Transformer
class TransformerConfig(object):
    def __init__(self, batch=32, len1=256, len2=256, d_model=512, heads=8, d_ff=2048, blocks=6, vocab=32000,
                 mask_value=-2.0 ** 32 + 1, smoothing=0.1, embed_std=None, pos_amplitude=1.0):
        self.batch, self.len1, self.len2, self.d_model, self.heads = batch, len1, len2, d_model, heads
        self.d_ff, self.blocks, self.vocab, self.mask_value, self.smoothing = d_ff, blocks, vocab, mask_value, smoothing
        # The graph has no softmax and no layer norm (as in the reference's example), so its
        # activations grow cubically per attention layer; the reference draws every variable,
        # the position table included, from N(0, 0.1) (examples/transformer.py:37-45).  Small
        # values here keep a deep stack finite.
        self.embed_std = d_model ** -0.5 if embed_std is None else embed_std
        self.pos_amplitude = pos_amplitude


def _dense(t, b, x, fan_in, fan_out, relu=False):
    """examples/transformer.py:56-69."""
    name = b.unique("dense")
    y = t.matmul(x, b.get(name + "_weight", (fan_in, fan_out), np.sqrt(1.0 / fan_in)))
    y = t.add_bias(y, b.get(name + "_bias", (fan_out,), "zero"))
    return t.relu(y) if relu else y


def _const_full(t, b, value, shape):
    one = b.constant(("scalar", float(value)), lambda: np.full((1,), value, np.float32))
    return t.broadcast_like(one, shape)


def _attention(t, b, cfg, queries, keys, values, mask_ids, causal):
    """examples/transformer.py:93-171: projections, head split, scaled scores, padding mask
    added, causal mask selected, scores x values (no softmax), head merge, residual."""
    N, h, d = cfg.batch, cfg.heads, cfg.d_model
    dh = d // h
    tq, tk = queries.shape[1], keys.shape[1]

    def heads(x2d, length):
        return t.transpose(t.reshape(x2d, (N, length, h, dh)), (0, 2, 1, 3))

    q = heads(_dense(t, b, t.reshape(queries, (-1, d)), d, d), tq)
    k = heads(_dense(t, b, t.reshape(keys, (-1, d)), d, d), tk)
    v = heads(_dense(t, b, t.reshape(values, (-1, d)), d, d), tk)
    scores = t.scale(t.batch_matmul(q, k, trans_b=True), 1.0 / np.sqrt(float(dh)))     # [N,h,tq,tk]
    if mask_ids is not None:
        zeros = _const_full(t, b, 0.0, mask_ids.shape)
        adder = _const_full(t, b, cfg.mask_value, mask_ids.shape)
        m = t.where(mask_ids, zeros, adder)                                             # [N,tk]
        m = t.reshape(m, (N, 1, 1, tk))
        scores = t.add(scores, t.broadcast_like(m, scores.shape))
    if causal:
        tril = b.constant(("tril", tq, tk), lambda: np.tril(np.ones((tq, tk), np.float32)))
        future = t.broadcast_like(tril, scores.shape)
        scores = t.where(future, scores, _const_full(t, b, cfg.mask_value, scores.shape))
    ctx = t.batch_matmul(scores, v)                                                     # [N,h,tq,dh]
    out = t.reshape(t.transpose(ctx, (0, 2, 1, 3)), (N, tq, d))
    return t.add(out, queries)


def _ffn(t, b, cfg, x):
    """examples/transformer.py:174-181."""
    y = _dense(t, b, t.reshape(x, (-1, cfg.d_model)), cfg.d_model, cfg.d_ff, relu=True)
    y = _dense(t, b, y, cfg.d_ff, cfg.d_model)
    return t.add(t.reshape(y, x.shape), x)


def _positions(t, b, ids, length, d, amplitude):
    """examples/transformer.py:189-212: sinusoids, zeroed where the token id is 0."""
    n = ids.shape[0]

    def table():
        pos = np.array([[p / np.power(10000.0, (i & -2) / float(d)) for i in range(d)] for p in range(length)])
        pos[:, 0::2] = np.sin(pos[:, 0::2])
        pos[:, 1::2] = np.cos(pos[:, 1::2])
        return np.tile((amplitude * pos[None]).astype(np.float32), (n, 1, 1))
    enc = b.constant(("pos", n, length, d, float(amplitude)), table)
    zeros = b.constant(("zeros", n, length, d), lambda: np.zeros((n, length, d), np.float32))
    cond = t.broadcast_like(t.reshape(ids, (n, length, 1)), (n, length, d))
    return t.where(cond, enc, zeros)


def transformer(t, b, cfg, xs, ys_in, ys_out):
    """examples/transformer.py:215-287.  xs [N,len1], ys_in / ys_out [N,len2] hold token ids as
    float32.  Returns (loss, logits [N*len2, vocab]); the 3-D logits of the reference are kept
    2-D for the loss (its CUDA loss averages over all rows but scales the gradient by
    1/shape[0]: src/ops/SoftmaxCrossEntropy.cu:47-52,120, so only 2-D logits are well defined)."""
    d = cfg.d_model
    table = b.get("embedding_table", (cfg.vocab, d), cfg.embed_std)

    def embed(ids, length):
        e = t.scale(t.embedding(table, ids), d ** 0.5)
        return t.add(e, _positions(t, b, ids, length, d, cfg.pos_amplitude))

    enc = embed(xs, cfg.len1)
    for _ in range(cfg.blocks):
        enc = _ffn(t, b, cfg, _attention(t, b, cfg, enc, enc, enc, xs, False))
    dec = embed(ys_in, cfg.len2)
    for _ in range(cfg.blocks):
        dec = _attention(t, b, cfg, dec, dec, dec, ys_in, True)
        dec = _attention(t, b, cfg, dec, enc, enc, xs, False)
        dec = _ffn(t, b, cfg, dec)
    logits = t.matmul(t.reshape(dec, (-1, d)), table, trans_b=True)                      # [N*len2, vocab]
    onehot = t.one_hot(t.reshape(ys_out, (-1,)), cfg.vocab)
    labels = t.shift(t.scale(onehot, 1.0 - cfg.smoothing), cfg.smoothing / cfg.vocab)   # :184-186
    return t.softmax_ce(logits, labels), logits


# ------------------------------------------------------------------ LSTM
def lstm(t, b, x, labels, dim_input=28, dim_hidden=128, classes=10, steps=28, std=0.1):
    """The reference's LSTM classifier (examples/LSTM.py:21-90): every row of x holds `steps`
    frames of `dim_input` values, cut out with slice; one LSTM cell with separate forget / input
    / output / candidate weights (W on the frame, U on the hidden state, bias broadcast); the
    last hidden state feeds a linear layer and softmax cross-entropy.  All variables ~ N(0, std)
    as the example draws them (LSTM.py:14-15).  Returns (loss, logits)."""
    gates = {}
    for g in ("forget_gate", "input_gate", "output_gate", "tanh"):
        gates[g] = (b.get("lstm_%s_w" % g, (dim_input, dim_hidden), std), b.get("lstm_%s_u" % g, (dim_hidden, dim_hidden), std),
                    b.get("lstm_%s_b" % g, (dim_hidden,), std))
    out_w = b.get("lstm_out_weight", (dim_hidden, classes), std)
    out_b = b.get("lstm_out_bias", (classes,), std)
    initial = b.get("initial_state", (1,), std, trainable=False)
    n = x.shape[0]

    def gate(name, frame, h, act):
        w, u, bias = gates[name]
        z = t.add(t.matmul(h, u), t.matmul(frame, w))
        z = t.add(z, t.broadcast_like(bias, z.shape))
        return act(z)

    c = h = None
    for i in range(steps):
        frame = t.slice(x, (0, i * dim_input), (-1, dim_input))
        if i == 0:
            c = t.broadcast_like(initial, (n, dim_hidden))
            h = t.broadcast_like(initial, (n, dim_hidden))
        f = gate("forget_gate", frame, h, t.sigmoid)
        ig = gate("input_gate", frame, h, t.sigmoid)
        o = gate("output_gate", frame, h, t.sigmoid)
        cand = gate("tanh", frame, h, t.tanh)
        c = t.add(t.mul(c, f), t.mul(ig, cand))
        h = t.mul(t.tanh(c), o)
    logits = t.matmul(h, out_w)
    logits = t.add(logits, t.broadcast_like(out_b, logits.shape))
    return t.softmax_ce(logits, labels), logits


# ------------------------------------------------------------------ shapes only
class _ShapeBackend(object):
    """Runs a builder without arithmetic: every primitive returns None; convolutions are listed."""

    def __init__(self):
        self.convs = []

    def conv2d(self, x, w, xs, ws, ph, pw, s):
        self.convs.append((int(xs[0]), int(xs[1]), int(xs[2]), int(xs[3]), int(ws[0]), int(ws[2]), int(ws[3]), int(ph),
                           int(pw), int(s)))

    def __getattr__(self, name):
        return lambda *a, **k: None


class _ShapeStore(object):
    trainable = {}

    def get(self, name, shape, init, trainable=True):
        return np.broadcast_to(np.float32(0), tuple(int(s) for s in shape))


def conv_geometries(net, batch=None):
    """The distinct convolution geometries of a full-size example network, in order of first use:
    tuples (images, Cin, H, W, Cout, kH, kW, pad_h, pad_w, stride).  net: "resnet50" (batch 64,
    224x224), "inception_v4" (batch 32, 299x299) or "vgg16" (batch 64, 224x224, the first four
    layers on a quarter of the batch each: the micro-tensors of the benchmark configuration,
    examples/imagenet_vgg.py:24-98), the sizes of the benchmark configurations."""
    from . import graph
    if net == "vgg16":
        from . import trainer
        n, hw, seen, out, ci = batch or 64, 224, set(), [], 0
        for layer in trainer.vgg16_spec():
            if layer[0] == "conv":
                _, _, cin, cout, k, pad, stride = layer
                g = ((n + 3) // 4 if ci < 4 else n, cin, hw, hw, cout, k, k, pad, pad, stride)
                ci += 1
                if g not in seen:
                    seen.add(g)
                    out.append(g)
            elif layer[0] == "maxpool":
                hw //= 2
        return out
    backend = _ShapeBackend()
    t = graph.Tape(backend)
    b = Binder(t, _ShapeStore())
    if net == "resnet50":
        n = batch or 64
        resnet(t, b, t.const(None, (n, 3, 224, 224)), t.const(None, (n, 1000)))
    elif net == "inception_v4":
        n = batch or 32
        inception_v4(t, b, t.const(None, (n, 3, 299, 299)), t.const(None, (n, 1000)))
    else:
        raise ValueError(net)
    seen, out = set(), []
    for g in backend.convs:
        if g not in seen:
            seen.add(g)
            out.append(g)
    return out
