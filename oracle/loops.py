"""CPU oracle, literal form: plain-loop statements of the reference's numpy
operator bodies, usable only on tiny shapes.

THIS IS TEST INFRASTRUCTURE (same rule as oracle/ops.py): tests use it to pin
the vectorised restatement in oracle/ops.py; nothing in the product imports it.

The loop nests keep the reference's iteration order (so accumulation order and
argmax tie-breaking are the reference's), with two stated generalisations:
output sizes floor instead of asserting divisibility, and conv takes separate
(pad_h, pad_w).
"""
import numpy as np


def _out(size, k, pad, stride):
    return (size + 2 * pad - k) // stride + 1


def im2col_loops(x, kH, kW, pad_h, pad_w, stride):
    """gpu_ops/Conv2d.py:34-61: for every image and output pixel, walk
    (c, y, x) taps in order and copy or zero-fill."""
    N, C, H, W = x.shape
    oH, oW = _out(H, kH, pad_h, stride), _out(W, kW, pad_w, stride)
    cols = np.empty((N, C * kH * kW, oH * oW), dtype=x.dtype)
    for n in range(N):
        for col in range(oH * oW):
            oy, ox = divmod(col, oW)
            y0, x0 = oy * stride - pad_h, ox * stride - pad_w
            row = 0
            for c in range(C):
                for yy in range(y0, y0 + kH):
                    for xx in range(x0, x0 + kW):
                        inside = 0 <= xx < W and 0 <= yy < H
                        cols[n, row, col] = x[n, c, yy, xx] if inside else 0
                        row += 1
    return cols


def conv2d_loops(x, w, pad_h, pad_w, stride):
    """gpu_ops/Conv2d.py:63-75."""
    O, I, kH, kW = w.shape
    N, C, H, W = x.shape
    oH, oW = _out(H, kH, pad_h, stride), _out(W, kW, pad_w, stride)
    cols = im2col_loops(x, kH, kW, pad_h, pad_w, stride)
    return np.matmul(w.reshape(O, -1), cols).reshape(N, O, oH, oW)


def conv2d_direct(x, w, pad_h, pad_w, stride):
    """Textbook 7-loop cross-correlation, independent of any im2col: the
    definition the im2col forms must reduce to."""
    O, I, kH, kW = w.shape
    N, C, H, W = x.shape
    oH, oW = _out(H, kH, pad_h, stride), _out(W, kW, pad_w, stride)
    y = np.zeros((N, O, oH, oW), dtype=np.float64)
    for n in range(N):
        for o in range(O):
            for oy in range(oH):
                for ox in range(oW):
                    acc = 0.0
                    for c in range(C):
                        for i in range(kH):
                            for j in range(kW):
                                yy, xx = oy * stride - pad_h + i, ox * stride - pad_w + j
                                if 0 <= yy < H and 0 <= xx < W:
                                    acc += float(x[n, c, yy, xx]) * float(w[o, c, i, j])
                    y[n, o, oy, ox] = acc
    return y


def col2im_loops(cols, N, C, H, W, kH, kW, pad_h, pad_w, stride):
    """gpu_ops/Conv2d.py:166-193: the im2col walk with += into the image."""
    oH, oW = _out(H, kH, pad_h, stride), _out(W, kW, pad_w, stride)
    dx = np.zeros((N, C, H, W), dtype=cols.dtype)
    for n in range(N):
        for col in range(oH * oW):
            oy, ox = divmod(col, oW)
            y0, x0 = oy * stride - pad_h, ox * stride - pad_w
            row = 0
            for c in range(C):
                for yy in range(y0, y0 + kH):
                    for xx in range(x0, x0 + kW):
                        if 0 <= xx < W and 0 <= yy < H:
                            dx[n, c, yy, xx] += cols[n, row, col]
                        row += 1
    return dx


def conv2d_grad_data_loops(w, dy, x_shape, pad_h, pad_w, stride):
    """gpu_ops/Conv2d.py:195-204."""
    O, I, kH, kW = w.shape
    N = dy.shape[0]
    dcols = np.matmul(w.reshape(O, -1).T, dy.reshape(N, O, -1))
    return col2im_loops(dcols, *x_shape, kH, kW, pad_h, pad_w, stride)


def conv2d_grad_filter_loops(x, dy, w_shape, pad_h, pad_w, stride):
    """gpu_ops/Conv2d.py:328-342."""
    O, I, kH, kW = w_shape
    N = x.shape[0]
    cols = im2col_loops(x, kH, kW, pad_h, pad_w, stride)
    dyy = dy.reshape(N, O, -1)
    dw = np.zeros((O, I * kH * kW), dtype=dy.dtype)
    for n in range(N):
        dw += np.matmul(dyy[n], cols[n].T)
    return dw.reshape(w_shape)


def max_pool_loops(x, kH, kW, pad, stride):
    """gpu_ops/MaxPool.py:8-38.  Returns (pooled float32, argmax as h*W+w)."""
    N, C, H, W = x.shape
    pH, pW = _out(H, kH, pad, stride), _out(W, kW, pad, stride)
    out = np.zeros((N, C, pH, pW), dtype=np.float32)
    arg = np.zeros((N, C, pH, pW), dtype=np.int64)
    for n in range(N):
        for c in range(C):
            for h in range(pH):
                for w in range(pW):
                    hs, ws = h * stride - pad, w * stride - pad
                    hend, wend = min(hs + kH, H), min(ws + kW, W)
                    hs, ws = max(hs, 0), max(ws, 0)
                    hm, wm = hs, ws
                    for i in range(hs, hend):
                        for j in range(ws, wend):
                            if x[n, c, i, j] > x[n, c, hm, wm]:
                                hm, wm = i, j
                    out[n, c, h, w] = x[n, c, hm, wm]
                    arg[n, c, h, w] = hm * W + wm
    return out, arg


def max_pool_grad_loops(x, dy, kH, kW, pad, stride):
    """gpu_ops/MaxPool.py:40-68 (float32 accumulator, window order)."""
    N, C, H, W = x.shape
    _, _, pH, pW = dy.shape
    dx = np.zeros((N, C, H, W), dtype=np.float32)
    for n in range(N):
        for c in range(C):
            for h in range(pH):
                for w in range(pW):
                    hs, ws = h * stride - pad, w * stride - pad
                    hend, wend = min(hs + kH, H), min(ws + kW, W)
                    hs, ws = max(hs, 0), max(ws, 0)
                    hm, wm = hs, ws
                    for i in range(hs, hend):
                        for j in range(ws, wend):
                            if x[n, c, i, j] > x[n, c, hm, wm]:
                                hm, wm = i, j
                    dx[n, c, hm, wm] += dy[n, c, h, w]
    return dx
