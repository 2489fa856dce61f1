"""CPU oracle: numpy restatement of the reference's CPU operator semantics.

THIS IS TEST INFRASTRUCTURE.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.  The product path (the C-ABI
library and the tsplit_amd package) never calls into this module.

Each function restates the numpy branch of one reference operator
(python/athena/gpu_ops/<Op>.py `compute(..., use_numpy=True)`), vectorised so it
finishes in seconds, and cites the reference lines it follows.  Literal
loop-for-loop transcriptions of the same bodies live in oracle/loops.py and are
used to pin these vectorised forms on tiny shapes.

Precision policy: operands are rounded to float32 first (what the GPU sees),
arithmetic runs in `dtype` (float64 by default, the reference's numpy path is
effectively float64: examples/imagenet_vgg.py:18, gpu_ops/executor.py:147).

Domain extensions over the reference numpy bodies (which assert exact
divisibility and take one padding int, gpu_ops/Conv2d.py:36-37,
gpu_ops/MaxPool.py:10-11): output sizes floor, and conv takes (pad_h, pad_w) as
the GPU symbols do (src/ops/CudnnConv2d.cu:154-157).

Parity status per function (what pins it, see tests/test_oracle*.py; conv, BN, the pools,
softmax-CE and a whole backward sweep are also checked against PyTorch-CPU autograd in
tests/test_oracle_vs_library.py):
  conv2d / conv2d_grad_data / conv2d_grad_filter  pinned: brute-force loops,
      scipy.signal.correlate2d, adjoint identities
  matmul                                           np.matmul is the reference
  batchnorm_forward                                pinned: closed form + invariants
  batchnorm_backward                               pinned: finite differences of
      batchnorm_forward, sum(dx)=0; NOT the reference's numpy body, which is
      defective (gpu_ops/BatchNorm.py:524-544 divides by the channel count and
      uses running averages); follows the standard batch-statistics formula the
      reference's GPU and dnnl paths implement (src/ops/CudnnBn.cu:367-375,
      src/dnnl_ops/BatchNorm.cpp:63-116)
  relu / relu_grad                                 pinned: closed form incl. x==0
  max_pool / max_pool_grad                         pinned: literal loops, tie cases
  softmax / softmax_ce / softmax_ce_grad           pinned: closed forms, invariants
  sgd / momentum / adagrad / adam                  pinned: hand-computed 3-step vectors
  split / concat / slice                           pinned: integer index arithmetic
  avg_pool / avg_pool_grad                         pinned: literal loops, depthwise
      correlation with a constant filter, adjoint identity
  broadcast_* / reduce_* / pad / transpose / one_hot / where / embedding_*
                                                   pinned: literal loops on small shapes
  batch_matmul                                     pinned: per-batch matmul loops
  sqrt / rsqrt / sigmoid / tanh / opposite / div_const / divide
                                                   pinned: inverse-function identities
  csrmv / csrmm                                    pinned: scipy.sparse products are the
      reference's CPU path; checked against dense float64 products and literal loops
  reduce_sum_axis_zero (workspace form)            same function as reduce_sum_axis_zero
  dropout / dropout_grad                           arithmetic pinned (kept elements scaled
      by 1/(1-p), dropped ones exactly 0, the gradient reuses the forward mask, the mask
      repeats from call to call because the reference re-seeds before every call);
      philox4x32_10 pinned by the published Random123 known-answer vectors.
      WHICH elements are dropped: PARITY UNPINNED.  The reference's GPU mask comes from
      cuDNN's generator (src/ops/CudnnDropout.cu:33-60, closed source, unversioned) and its
      CPU paths use libc rand() (src/dnnl_ops/Dropout.cpp:17-31) or numpy's global
      generator (gpu_ops/Dropout.py:64-67); no reference test or fixture fixes a mask.
"""
import numpy as np

F32 = np.float32


def _f(a, dtype):
    """Round to float32 (what the device holds), then widen to the compute dtype."""
    return np.asarray(a, dtype=F32).astype(dtype)


# --------------------------------------------------------------------------
# Conv2d  (reference: gpu_ops/Conv2d.py:34-75 fwd, :166-204 bwd-data, :297-342 bwd-filter)
# --------------------------------------------------------------------------
def conv_out_size(size, k, pad, stride):
    """Floor semantics of the GPU path (cuDNN); equals the numpy body
    (gpu_ops/Conv2d.py:38-39) whenever that body's divisibility assert holds."""
    return (size + 2 * pad - k) // stride + 1


def im2col(x, kH, kW, pad_h, pad_w, stride):
    """[N,C,H,W] -> [N, C*kH*kW, oH*oW]; row index runs (c, kh, kw), column index
    runs (oh, ow); out-of-image taps are 0 (gpu_ops/Conv2d.py:34-61)."""
    N, C, H, W = x.shape
    oH = conv_out_size(H, kH, pad_h, stride)
    oW = conv_out_size(W, kW, pad_w, stride)
    xp = np.pad(x, ((0, 0), (0, 0), (pad_h, pad_h), (pad_w, pad_w)))
    win = np.lib.stride_tricks.sliding_window_view(xp, (kH, kW), axis=(2, 3))
    win = win[:, :, ::stride, ::stride][:, :, :oH, :oW]        # N,C,oH,oW,kH,kW
    cols = win.transpose(0, 1, 4, 5, 2, 3).reshape(N, C * kH * kW, oH * oW)
    return np.ascontiguousarray(cols)


def conv2d(x, w, pad_h=0, pad_w=None, stride=1, dtype=np.float64):
    """y = x (*) w, cross-correlation, no bias: filter matrix @ im2col
    (gpu_ops/Conv2d.py:63-75)."""
    if pad_w is None:
        pad_w = pad_h
    x = _f(x, dtype)
    w = _f(w, dtype)
    N, C, H, W = x.shape
    O, I, kH, kW = w.shape
    assert I == C
    oH = conv_out_size(H, kH, pad_h, stride)
    oW = conv_out_size(W, kW, pad_w, stride)
    cols = im2col(x, kH, kW, pad_h, pad_w, stride)
    y = np.matmul(w.reshape(O, -1), cols)
    return y.reshape(N, O, oH, oW)


def col2im(cols, x_shape, kH, kW, pad_h, pad_w, stride):
    """Scatter-add transpose of im2col (gpu_ops/Conv2d.py:166-193)."""
    N, C, H, W = x_shape
    oH = conv_out_size(H, kH, pad_h, stride)
    oW = conv_out_size(W, kW, pad_w, stride)
    cols = cols.reshape(N, C, kH, kW, oH, oW)
    dxp = np.zeros((N, C, H + 2 * pad_h, W + 2 * pad_w), dtype=cols.dtype)
    for kh in range(kH):
        for kw in range(kW):
            dxp[:, :, kh:kh + stride * oH:stride, kw:kw + stride * oW:stride] += cols[:, :, kh, kw]
    return dxp[:, :, pad_h:pad_h + H, pad_w:pad_w + W]


def conv2d_grad_data(w, dy, x_shape, pad_h=0, pad_w=None, stride=1, dtype=np.float64):
    """dx = col2im(F^T @ dY)  (gpu_ops/Conv2d.py:195-204).  x_shape comes from the
    caller because flooring makes it ambiguous for stride > 1 (the reference takes
    it from the pre-allocated output array)."""
    if pad_w is None:
        pad_w = pad_h
    w = _f(w, dtype)
    dy = _f(dy, dtype)
    O, I, kH, kW = w.shape
    N = dy.shape[0]
    dcols = np.matmul(w.reshape(O, -1).T, dy.reshape(N, O, -1))
    return np.ascontiguousarray(col2im(dcols, x_shape, kH, kW, pad_h, pad_w, stride))


def conv2d_grad_filter(x, dy, w_shape, pad_h=0, pad_w=None, stride=1, dtype=np.float64):
    """dw = sum_n dY[n] @ im2col(x)[n]^T  (gpu_ops/Conv2d.py:328-342)."""
    if pad_w is None:
        pad_w = pad_h
    x = _f(x, dtype)
    dy = _f(dy, dtype)
    O, I, kH, kW = w_shape
    N = x.shape[0]
    cols = im2col(x, kH, kW, pad_h, pad_w, stride)
    dw = np.zeros((O, I * kH * kW), dtype=dtype)
    dyy = dy.reshape(N, O, -1)
    for n in range(N):
        dw += np.matmul(dyy[n], cols[n].T)
    return dw.reshape(O, I, kH, kW)


# --------------------------------------------------------------------------
# MatMul  (reference: gpu_ops/MatrixMult.py:58-86)
# --------------------------------------------------------------------------
def matmul(A, transA, B, transB, dtype=np.float64):
    A = _f(A, dtype)
    B = _f(B, dtype)
    if transA:
        A = A.T
    if transB:
        B = B.T
    return np.matmul(A, B)


# --------------------------------------------------------------------------
# BatchNorm  (reference fwd: gpu_ops/BatchNorm.py:503-521)
# --------------------------------------------------------------------------
def batchnorm_forward(x, scale, bias, eps=0.01, dtype=np.float64):
    """Training-mode spatial BN with biased batch variance.  Returns
    (y, batch_mean, batch_var).  The reference's running-average outputs
    (BatchNorm.py:512-513) are thrown away on its GPU path
    (src/ops/CudnnBn.cu:164-176) and are not part of the contract."""
    x = _f(x, dtype)
    D = x.shape[1]
    g = _f(scale, dtype).reshape(1, D, 1, 1)
    b = _f(bias, dtype).reshape(1, D, 1, 1)
    mean = x.mean(axis=(0, 2, 3))
    var = x.var(axis=(0, 2, 3))
    std = np.sqrt(var.reshape(1, D, 1, 1) + eps)
    y = g * ((x - mean.reshape(1, D, 1, 1)) / std) + b
    return y, mean, var


def batchnorm_backward(dy, x, scale, eps=0.01, dtype=np.float64):
    """Standard batch-statistics BN gradient (statistics recomputed from x, as
    the reference's GPU path does when saved stats are NULL:
    gpu_ops/BatchNorm.py:224-227 -> src/ops/CudnnBn.cu:367-375).
    Returns (dx, dscale, dbias); dscale/dbias have shape [C]."""
    dy = _f(dy, dtype)
    x = _f(x, dtype)
    D = x.shape[1]
    g = _f(scale, dtype).reshape(1, D, 1, 1)
    m = x.shape[0] * x.shape[2] * x.shape[3]
    mean = x.mean(axis=(0, 2, 3)).reshape(1, D, 1, 1)
    var = x.var(axis=(0, 2, 3)).reshape(1, D, 1, 1)
    inv_std = 1.0 / np.sqrt(var + eps)
    xhat = (x - mean) * inv_std
    dbias = dy.sum(axis=(0, 2, 3))
    dscale = (dy * xhat).sum(axis=(0, 2, 3))
    dx = g * inv_std * (dy - dbias.reshape(1, D, 1, 1) / m - xhat * dscale.reshape(1, D, 1, 1) / m)
    return dx, dscale, dbias


# --------------------------------------------------------------------------
# Relu  (reference: gpu_ops/Relu.py:51,117)
# --------------------------------------------------------------------------
def relu(x, dtype=np.float64):
    return np.maximum(_f(x, dtype), 0)


def relu_grad(x, dy, dtype=np.float64):
    """(sign(x)+1)*0.5*dy: 0.5*dy at x == 0 (numpy and CUDA bodies agree)."""
    return (np.sign(_f(x, dtype)) + 1) * 0.5 * _f(dy, dtype)


# --------------------------------------------------------------------------
# MaxPool  (reference: gpu_ops/MaxPool.py:8-68)
# --------------------------------------------------------------------------
def max_pool_argmax(x, kH, kW, pad=0, stride=1):
    """Flat input index (h*W + w) of the first strict maximum of each window in
    row-major (h, then w) scan order; windows are clipped to the image
    (gpu_ops/MaxPool.py:21-35).  Integer result, dtype-independent."""
    x = np.asarray(x, dtype=F32)
    N, C, H, W = x.shape
    pH = conv_out_size(H, kH, pad, stride)
    pW = conv_out_size(W, kW, pad, stride)
    best_v = np.full((N, C, pH, pW), -np.inf, dtype=F32)
    best_i = np.full((N, C, pH, pW), -1, dtype=np.int64)
    oh = np.arange(pH)[:, None]
    ow = np.arange(pW)[None, :]
    for i in range(kH):
        for j in range(kW):
            ih = oh * stride - pad + i          # [pH,1]
            iw = ow * stride - pad + j          # [1,pW]
            ok = (ih >= 0) & (ih < H) & (iw >= 0) & (iw < W)
            ihc = np.clip(ih, 0, H - 1)
            iwc = np.clip(iw, 0, W - 1)
            v = x[:, :, ihc, iwc]               # N,C,pH,pW
            first = ok & (best_i < 0)           # initial candidate = first in-image tap
            take = ok & ((v > best_v) | first)
            best_v = np.where(take, v, best_v)
            best_i = np.where(take, np.broadcast_to(ihc * W + iwc, v.shape), best_i)
    return best_i


def max_pool(x, kH, kW, pad=0, stride=1):
    """Pooled values (float32 copies of inputs, exact)."""
    x = np.asarray(x, dtype=F32)
    N, C, H, W = x.shape
    idx = max_pool_argmax(x, kH, kW, pad, stride)
    flat = x.reshape(N, C, H * W)
    return np.take_along_axis(flat, idx.reshape(N, C, -1), axis=2).reshape(idx.shape)


def max_pool_grad(x, dy, kH, kW, pad=0, stride=1, dtype=np.float64):
    """dx[argmax] += dy, accumulated in window order (gpu_ops/MaxPool.py:40-68).
    dx has the shape of x (the reference derives it from dy; identical when the
    divisibility assert holds)."""
    x = np.asarray(x, dtype=F32)
    dy = _f(dy, dtype)
    N, C, H, W = x.shape
    idx = max_pool_argmax(x, kH, kW, pad, stride).reshape(N * C, -1)
    dx = np.zeros((N * C, H * W), dtype=dtype)
    dyf = dy.reshape(N * C, -1)
    rows = np.arange(N * C)
    for p in range(idx.shape[1]):               # window order => same accumulation order
        dx[rows, idx[:, p]] += dyf[:, p]
    return dx.reshape(N, C, H, W)


# --------------------------------------------------------------------------
# Softmax / SoftmaxCrossEntropy  (reference: gpu_ops/Softmax.py:7-12,
# gpu_ops/SoftmaxCrossEntropy.py:60-67,134-135)
# --------------------------------------------------------------------------
def softmax(y, dtype=np.float64):
    y = _f(y, dtype)
    b = y - np.max(y, axis=1, keepdims=True)
    e = np.exp(b)
    return e / np.sum(e, axis=1, keepdims=True)


def softmax_ce(y, y_, dtype=np.float64):
    """mean over rows of -sum(y_ * log(softmax(y))); shape (1,).  Evaluated in
    log-sum-exp form (as src/ops/SoftmaxCrossEntropy.cu:27 does): identical in
    exact arithmetic to log(softmax), and free of the underflow -> log(0) the
    literal numpy form hits for very negative logits."""
    y = _f(y, dtype)
    y_ = _f(y_, dtype)
    b = y - np.max(y, axis=1, keepdims=True)
    logsm = b - np.log(np.sum(np.exp(b), axis=1, keepdims=True))
    return np.mean(-np.sum(y_ * logsm, axis=1), keepdims=True)


def softmax_ce_grad(y, y_, g, dtype=np.float64):
    """(softmax(y) - y_) * g / y.shape[0]; g is the (1,) upstream gradient."""
    g = _f(g, dtype).reshape(-1)[0]
    return (softmax(y, dtype) - _f(y_, dtype)) * g / np.asarray(y).shape[0]


# --------------------------------------------------------------------------
# Optimizers  (reference: optimizer.py:119,170-176,225-227,286-290;
# fp32 evaluation order in src/ops/Optimizers.cu:3-7,33-46,80-85,112-120)
# --------------------------------------------------------------------------
def sgd_update(p, g, lr, dtype=np.float64):
    return _f(p, dtype) - lr * _f(g, dtype)


def momentum_update(p, g, v, lr, momentum, nesterov=False, dtype=np.float64):
    p, g, v = _f(p, dtype), _f(g, dtype), _f(v, dtype)
    if nesterov:
        lr_g = -lr * g
        v = momentum * (v + lr_g)
        p = p + v + lr_g
    else:
        v = momentum * v - lr * g
        p = p + v
    return p, v


def adagrad_update(p, g, acc, lr, eps, dtype=np.float64):
    p, g, acc = _f(p, dtype), _f(g, dtype), _f(acc, dtype)
    acc = acc + g * g
    p = p - lr * g / (np.sqrt(acc) + eps)
    return p, acc


def adam_update(p, g, m, v, lr, beta1, beta2, beta1t, beta2t, eps, dtype=np.float64):
    """beta1t/beta2t are the already-advanced powers beta^t (optimizer.py:254-255)."""
    p, g, m, v = _f(p, dtype), _f(g, dtype), _f(m, dtype), _f(v, dtype)
    m = beta1 * m + (1 - beta1) * g
    v = beta2 * v + (1 - beta2) * g * g
    mc = m / (1 - beta1t)
    vc = v / (1 - beta2t)
    p = p - lr * mc / (np.sqrt(vc) + eps)
    return p, m, v


# --------------------------------------------------------------------------
# Micro-tensor split  (reference: ndarray.py:390-409, src/common/c_runtime_api.cc:212-271,
# :164-210) -- integer arithmetic only
# --------------------------------------------------------------------------
def split_shape(shape, total, dimension=0):
    """Shapes of the `total` pieces: the first shape[d] % total pieces get one extra."""
    d = dimension
    base, extra = shape[d] // total, shape[d] % total
    out = []
    for i in range(total):
        s = list(shape)
        s[d] = base + (1 if i < extra else 0)
        out.append(tuple(s))
    return out


def micro_tensor_view(shape, total, index, dimension=0):
    """(element offset, shape) of piece `index`.  For dimension 0 this is a true
    batch slice.  For dimension 1 the reference re-labels a contiguous chunk as
    [N, C/total, ...] (c_runtime_api.cc:247-268): a true channel slice only when
    N == 1; restated as is."""
    d = 0 if dimension == 0 else 1
    size = int(np.prod(shape))
    D = shape[d]
    length = size // D
    base, extra = D // total, D % total
    off = 0
    for i in range(1, index + 1):
        off += (base + 1) * length if i <= extra else base * length
    s = list(shape)
    s[d] = base + (1 if index < extra else 0)
    return off, tuple(s)


def reuse_alloc_layout(in_shape, out_shape, pieces, overlap):
    """(total bytes, input byte offset, output byte offset) of the overlapped
    in/out buffer: output at the base, input flush with the end
    (c_runtime_api.cc:170-203)."""
    in_b = int(np.prod(in_shape)) * 4
    out_b = int(np.prod(out_shape)) * 4
    total = out_b + in_b // pieces * (pieces - overlap)
    return total, total - in_b, 0


# --------------------------------------------------------------------------
# Concat / Slice  (reference: gpu_ops/Concat.py:60,184-199, gpu_ops/Slice.py:56,136)
# --------------------------------------------------------------------------
def concat(a, b, axis=0):
    return np.concatenate((np.asarray(a, F32), np.asarray(b, F32)), axis=axis)


def concat_grad(dout, in_shape, axis=0, idx=0):
    """Slice of dout that belongs to input `idx` (0: leading, 1: trailing)."""
    dout = np.asarray(dout, F32)
    n = in_shape[axis]
    sl = [slice(None)] * dout.ndim
    sl[axis] = slice(0, n) if idx == 0 else slice(dout.shape[axis] - n, dout.shape[axis])
    return np.ascontiguousarray(dout[tuple(sl)])


def slice_(x, begin, out_shape):
    x = np.asarray(x, F32)
    sl = tuple(slice(b, b + s) for b, s in zip(begin, out_shape))
    return np.ascontiguousarray(x[sl])


def slice_grad(dy, begin, out_shape):
    """Zero tensor of out_shape with dy written at `begin` (gpu_ops/Slice.py:136)."""
    dy = np.asarray(dy, F32)
    out = np.zeros(out_shape, dtype=F32)
    sl = tuple(slice(b, b + s) for b, s in zip(begin, dy.shape))
    out[sl] = dy
    return out


# --------------------------------------------------------------------------
# Graph-closure elementwise ops  (reference: gpu_ops/AddElewise.py, AddConst.py,
# MultiplyConst.py, MultiplyElewise.py, OnesLike.py, ZerosLike.py, Reshape.py:64-90)
# --------------------------------------------------------------------------
def add(a, b, dtype=np.float64):
    return _f(a, dtype) + _f(b, dtype)


def add_const(a, c, dtype=np.float64):
    return _f(a, dtype) + dtype(F32(c))


def mul_const(a, c, dtype=np.float64):
    return _f(a, dtype) * dtype(F32(c))


def mul(a, b, dtype=np.float64):
    return _f(a, dtype) * _f(b, dtype)


def array_set(shape, value):
    return np.full(shape, F32(value), dtype=F32)


def reshape(a, shape):
    return np.asarray(a, F32).reshape(shape)


# --------------------------------------------------------------------------
# AvgPool  (reference: gpu_ops/AvgPool.py:27-50 fwd, :139-161 bwd)
# --------------------------------------------------------------------------
def avg_pool(x, kH, kW, pad=0, stride=1, dtype=np.float64):
    """Sum over the window clipped to the image, divided by kH*kW whatever the
    clipping (padding counts as zeros in the mean)."""
    x = _f(x, dtype)
    N, C, H, W = x.shape
    pH, pW = conv_out_size(H, kH, pad, stride), conv_out_size(W, kW, pad, stride)
    xp = np.zeros((N, C, H + 2 * pad + kH, W + 2 * pad + kW), dtype=dtype)   # slack for floor-sized outputs
    xp[:, :, pad:pad + H, pad:pad + W] = x
    y = np.zeros((N, C, pH, pW), dtype=dtype)
    for i in range(kH):
        for j in range(kW):
            y += xp[:, :, i:i + (pH - 1) * stride + 1:stride, j:j + (pW - 1) * stride + 1:stride]
    return y / (kH * kW)


def avg_pool_grad(dy, x_shape, kH, kW, pad=0, stride=1, dtype=np.float64):
    """Every in-image element of a window receives dy/(kH*kW)."""
    dy = _f(dy, dtype)
    N, C, H, W = x_shape
    pH, pW = dy.shape[2], dy.shape[3]
    dxp = np.zeros((N, C, H + 2 * pad + kH, W + 2 * pad + kW), dtype=dtype)
    g = dy / (kH * kW)
    for i in range(kH):
        for j in range(kW):
            dxp[:, :, i:i + (pH - 1) * stride + 1:stride, j:j + (pW - 1) * stride + 1:stride] += g
    return dxp[:, :, pad:pad + H, pad:pad + W].copy()


# --------------------------------------------------------------------------
# Broadcast / reduce  (reference: gpu_ops/Broadcast.py:59, ReduceSumAxisZero.py:55,
# Conv2dBroadcast.py:54-55, Conv2dReduceSum.py:48, BroadcastShape.py:52-56,
# ReduceSum.py:58-64)
# --------------------------------------------------------------------------
def broadcast_to(x, shape, dtype=np.float64):
    """numpy broadcasting of x against `shape` (new leading axes)."""
    return np.broadcast_to(_f(x, dtype), shape).copy()


def reduce_sum_axis_zero(x, dtype=np.float64):
    return np.sum(_f(x, dtype), axis=0)


def conv2d_broadcast_to(bias, shape, dtype=np.float64):
    """bias [C] -> [N,C,H,W] with out[n,c,h,w] = bias[c] (src/ops/Conv2dBroadcast.cu:4-10)."""
    b = _f(bias, dtype)
    assert b.shape == (shape[1],)
    return np.broadcast_to(b.reshape(1, -1, 1, 1), shape).copy()


def conv2d_reduce_sum(x, dtype=np.float64):
    return np.sum(_f(x, dtype), axis=(0, 2, 3))


def broadcast_shape(x, shape, add_axes=None, dtype=np.float64):
    """With add_axes: x's axes are placed at the positions of `shape` not listed in
    add_axes, the listed ones are new; without: numpy alignment from the right
    (src/ops/BroadcastShape.cu:23-63)."""
    x = _f(x, dtype)
    if add_axes:
        in_shape = list(shape)
        for a in add_axes:
            in_shape[a] = 1
        rest = [i for i in range(len(shape)) if i not in set(add_axes)]
        assert len(rest) == x.ndim
        for i, a in enumerate(rest):
            in_shape[a] = x.shape[i]
        x = x.reshape(in_shape)
    return np.broadcast_to(x, shape).copy()


def reduce_sum(x, axes, keepdims=False, dtype=np.float64):
    return np.sum(_f(x, dtype), axis=tuple(axes), keepdims=keepdims)


# --------------------------------------------------------------------------
# Pad  (reference: gpu_ops/Pad.py:194-203; CONSTANT mode, paddings for the last
# len(paddings) axes of a 4-D tensor: gpu_ops/Pad.py:73-80)
# --------------------------------------------------------------------------
def _full_paddings(paddings, ndim=4):
    paddings = [tuple(p) for p in paddings]
    return [(0, 0)] * (ndim - len(paddings)) + paddings


def pad(x, paddings, constant=0.0, dtype=np.float64):
    x = _f(x, dtype)
    return np.pad(x, _full_paddings(paddings, x.ndim), mode="constant", constant_values=(constant, constant))


def pad_grad(dy, paddings, dtype=np.float64):
    dy = _f(dy, dtype)
    sl = tuple(slice(lo, dy.shape[i] - hi) for i, (lo, hi) in enumerate(_full_paddings(paddings, dy.ndim)))
    return dy[sl].copy()


# --------------------------------------------------------------------------
# BatchMatMul / Transpose  (reference: gpu_ops/BatchMatrixMult.py:50-75, Transpose.py:55)
# --------------------------------------------------------------------------
def batch_matmul(A, transA, B, transB, dtype=np.float64):
    A, B = _f(A, dtype), _f(B, dtype)
    if transA:
        A = np.swapaxes(A, -1, -2)
    if transB:
        B = np.swapaxes(B, -1, -2)
    return np.matmul(A, B)


def transpose(x, perm):
    return np.ascontiguousarray(np.transpose(np.asarray(x, dtype=F32), perm))


# --------------------------------------------------------------------------
# OneHot / Where / Embedding  (reference: gpu_ops/OneHot.py:44-46, Where.py:44,
# EmbeddingLookUp.py:41-42)
# --------------------------------------------------------------------------
def one_hot(ids, num_classes):
    ids = np.asarray(ids, dtype=F32)
    return (ids[..., None] == np.arange(num_classes, dtype=F32)).astype(F32)


def where(cond, a, b):
    return np.where(np.asarray(cond, dtype=F32) != 0, np.asarray(a, dtype=F32), np.asarray(b, dtype=F32))


def embedding_lookup(table, ids):
    """out[..., :] = table[int(ids[...]), :].  The numpy branch is followed; the CUDA
    kernel of the reference ignores ids (src/ops/EmbeddingLookup.cu:6-7 uses the row
    number instead), which cannot be what a lookup means."""
    table = np.asarray(table, dtype=F32)
    idx = np.asarray(ids, dtype=F32).astype(np.int64)
    return table[idx.reshape(-1)].reshape(idx.shape + (table.shape[1],))


def embedding_lookup_grad(dy, ids, table_shape, dtype=np.float64):
    """Scatter-add of the output gradient rows into a zeroed table gradient
    (src/ops/EmbeddingLookup.cu:56-65 with ids honoured)."""
    dy = _f(dy, dtype)
    idx = np.asarray(ids, dtype=F32).astype(np.int64).reshape(-1)
    g = np.zeros(table_shape, dtype=dtype)
    np.add.at(g, idx, dy.reshape(-1, table_shape[1]))
    return g


# --------------------------------------------------------------------------
# Elementwise math  (reference: gpu_ops/Sqrt.py, Sigmoid.py, Tanh.py, Opposite.py,
# Division.py; src/ops/DivideConst.cu:6 divides the constant BY the tensor)
# --------------------------------------------------------------------------
def sqrt(x, dtype=np.float64):
    return np.sqrt(_f(x, dtype))


def rsqrt(x, dtype=np.float64):
    return 1.0 / np.sqrt(_f(x, dtype))


def sigmoid(x, dtype=np.float64):
    return 1.0 / (1.0 + np.exp(-_f(x, dtype)))


def tanh(x, dtype=np.float64):
    return np.tanh(_f(x, dtype))


def opposite(x, dtype=np.float64):
    return -_f(x, dtype)


def div_const(c, x, dtype=np.float64):
    return dtype(F32(c)) / _f(x, dtype)


def divide(a, b, dtype=np.float64):
    return _f(a, dtype) / _f(b, dtype)


# --------------------------------------------------------------------------
# Sparse products  (reference: gpu_ops/CuSparse.py:52-59 csrmv, :147-163 csrmm; the GPU
# symbols take the three CSR arrays, src/ops/CuSparseCsrmv.cu:3-47, CuSparseCsrmm.cu:34-96)
# --------------------------------------------------------------------------
def _csr(data, indptr, indices, nrow, ncol, dtype):
    import scipy.sparse
    return scipy.sparse.csr_matrix((_f(data, dtype), np.asarray(indices, dtype=np.int32),
                                    np.asarray(indptr, dtype=np.int32)), shape=(nrow, ncol))


def csrmv(data, indptr, indices, nrow, ncol, trans, x, dtype=np.float64):
    """y = A x, or A^T x when `trans` (gpu_ops/CuSparse.py:55-58)."""
    A = _csr(data, indptr, indices, nrow, ncol, dtype)
    return (A.T if trans else A).dot(_f(x, dtype))


def csrmm(data, indptr, indices, nrow, ncol, transA, B, transB, dtype=np.float64):
    """C = op(A) op(B), all dense operands row-major (gpu_ops/CuSparse.py:150-163)."""
    A = _csr(data, indptr, indices, nrow, ncol, dtype)
    Bm = _f(B, dtype)
    return (A.T if transA else A).dot(Bm.T if transB else Bm)


# --------------------------------------------------------------------------
# Dropout  (reference GPU symbol: src/ops/CudnnDropout.cu:4-77 forward, :79-151 gradient)
# --------------------------------------------------------------------------
DROPOUT_SEED = 19260817          # src/ops/CudnnDropout.cu:33 (set again before every call)

_PHILOX_M0, _PHILOX_M1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
_PHILOX_W0, _PHILOX_W1 = 0x9E3779B9, 0xBB67AE85
_MASK32 = np.uint64(0xFFFFFFFF)


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Philox-4x32 with 10 rounds (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
    SC'11).  Counters are uint32 arrays (or scalars), the key two uint32 scalars; returns the four
    output words as uint32 arrays."""
    c = [np.asarray(v, dtype=np.uint64) for v in (c0, c1, c2, c3)]
    k0, k1 = int(k0) & 0xFFFFFFFF, int(k1) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _PHILOX_M0 * c[0]
        p1 = _PHILOX_M1 * c[2]
        c = [(p1 >> np.uint64(32)) ^ c[1] ^ np.uint64(k0), p1 & _MASK32,
             (p0 >> np.uint64(32)) ^ c[3] ^ np.uint64(k1), p0 & _MASK32]
        k0, k1 = (k0 + _PHILOX_W0) & 0xFFFFFFFF, (k1 + _PHILOX_W1) & 0xFFFFFFFF
    return [v.astype(np.uint32) for v in c]


def dropout_mask(n, dropout, seed=DROPOUT_SEED):
    """keep[i] for i < n.  Element i takes word i%4 of philox4x32_10(counter=(i//4,0,0,0),
    key=(seed low, seed high)) and is kept iff word >= floor(dropout * 2^32): a fraction
    `dropout` of the words lies below the threshold."""
    groups = (n + 3) // 4
    idx = np.arange(groups, dtype=np.uint64)
    zero = np.zeros(groups, dtype=np.uint64)
    words = philox4x32_10(idx & _MASK32, idx >> np.uint64(32), zero, zero, seed & 0xFFFFFFFF, seed >> 32)
    flat = np.stack(words, axis=1).reshape(-1)[:n].astype(np.uint64)
    threshold = np.uint64(min(int(float(np.float32(dropout)) * 4294967296.0), 1 << 32))
    return flat >= threshold


def dropout(x, dropout, dtype=np.float64):
    """-> (y, keep).  cuDNN semantics of the GPU symbol: each element is zeroed with probability
    `dropout`, the others are multiplied by 1/(1-dropout) (src/ops/CudnnDropout.cu:41,58-60)."""
    xv = _f(x, dtype)
    keep = dropout_mask(xv.size, dropout).reshape(xv.shape)
    with np.errstate(divide="ignore", invalid="ignore"):       # dropout == 1: nothing is kept
        scale = F32(1.0) / (F32(1.0) - F32(dropout))
        return np.where(keep, xv * dtype(scale), dtype(0)), keep


def dropout_grad(dy, dropout, keep, dtype=np.float64):
    """dx = dy * keep / (1-dropout) with the forward call's mask (src/ops/CudnnDropout.cu:130-132)."""
    with np.errstate(divide="ignore", invalid="ignore"):
        scale = F32(1.0) / (F32(1.0) - F32(dropout))
        return np.where(keep, _f(dy, dtype) * dtype(scale), dtype(0))
