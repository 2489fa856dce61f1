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


def avg_pool_loops(x, kH, kW, pad, stride):
    """gpu_ops/AvgPool.py:27-50."""
    N, C, H, W = x.shape
    pH, pW = _out(H, kH, pad, stride), _out(W, kW, pad, stride)
    y = np.zeros((N, C, pH, pW), dtype=np.float64)
    for n in range(N):
        for c in range(C):
            for h in range(pH):
                for w in range(pW):
                    hs, ws = h * stride - pad, w * stride - pad
                    he, we = min(hs + kH, H), min(ws + kW, W)
                    hs, ws = max(hs, 0), max(ws, 0)
                    for i in range(hs, he):
                        for j in range(ws, we):
                            y[n, c, h, w] += x[n, c, i, j]
                    y[n, c, h, w] /= kH * kW
    return y


def avg_pool_grad_loops(dy, x_shape, kH, kW, pad, stride):
    """gpu_ops/AvgPool.py:139-161."""
    N, C, H, W = x_shape
    pH, pW = dy.shape[2], dy.shape[3]
    dx = np.zeros(x_shape, dtype=np.float64)
    for n in range(N):
        for c in range(C):
            for h in range(pH):
                for w in range(pW):
                    hs, ws = h * stride - pad, w * stride - pad
                    he, we = min(hs + kH, H), min(ws + kW, W)
                    hs, ws = max(hs, 0), max(ws, 0)
                    for i in range(hs, he):
                        for j in range(ws, we):
                            dx[n, c, i, j] += dy[n, c, h, w] / (kH * kW)
    return dx


def broadcast_flat_loops(x, out_shape):
    """src/ops/Broadcast.cu:4-9: out[id] = in[id % in_size]."""
    flat = np.asarray(x).reshape(-1)
    out = np.empty(int(np.prod(out_shape)), dtype=flat.dtype)
    for i in range(out.size):
        out[i] = flat[i % flat.size]
    return out.reshape(out_shape)


def broadcast_shape_loops(x, out_shape, add_axes=None):
    """src/ops/BroadcastShape.cu:4-63: host builds in_dims (1 where an axis is new or
    broadcast), the kernel walks the output index and skips axes of extent 1."""
    x = np.asarray(x)
    nd = len(out_shape)
    diff = nd - x.ndim
    in_dims = [0] * nd
    if add_axes is None:
        for i in range(nd):
            in_dims[i] = 1 if i < diff else x.shape[i - diff]
    else:
        for a in add_axes[:diff]:
            in_dims[a] = 1
        o = 0
        for i in range(x.ndim):
            while in_dims[o] == 1:
                o += 1
            in_dims[o] = x.shape[i]
            o += 1
    strides = [int(np.prod(out_shape[i + 1:])) for i in range(nd)]
    flat = x.reshape(-1)
    out = np.empty(int(np.prod(out_shape)), dtype=x.dtype)
    for o_ind in range(out.size):
        i_ind, t = 0, o_ind
        for i in range(nd):
            i_ind *= in_dims[i]
            q = t // strides[i]
            if in_dims[i] > 1:
                i_ind += q
            t %= strides[i]
        out[o_ind] = flat[i_ind]
    return out.reshape(out_shape)


def pad_loops(x, paddings, constant):
    """src/ops/Pad.cu:4-18 with np.pad's treatment of the unpadded leading axes
    (gpu_ops/Pad.py:194-196): each output element is either the shifted input element
    or the constant."""
    full = [(0, 0)] * (x.ndim - len(paddings)) + [tuple(p) for p in paddings]
    out_shape = tuple(x.shape[i] + full[i][0] + full[i][1] for i in range(x.ndim))
    out = np.empty(out_shape, dtype=x.dtype)
    for idx in np.ndindex(*out_shape):
        src = tuple(idx[i] - full[i][0] for i in range(x.ndim))
        inside = all(0 <= src[i] < x.shape[i] for i in range(x.ndim))
        out[idx] = x[src] if inside else constant
    return out


def transpose_loops(x, perm):
    """src/ops/Transpose.cu:3-17: out[o] = in[sum_d coord_d(o) * in_stride[perm[d]]]."""
    out_shape = tuple(x.shape[p] for p in perm)
    out = np.empty(out_shape, dtype=x.dtype)
    for idx in np.ndindex(*out_shape):
        src = [0] * x.ndim
        for d, p in enumerate(perm):
            src[p] = idx[d]
        out[idx] = x[tuple(src)]
    return out


def batch_matmul_loops(A, transA, B, transB):
    """One 2-D product per leading index (src/ops/BatchMatrixMult.cu: strided batched GEMM)."""
    lead = A.shape[:-2]
    A2 = A.reshape((-1,) + A.shape[-2:]).astype(np.float64)
    B2 = B.reshape((-1,) + B.shape[-2:]).astype(np.float64)
    outs = []
    for b in range(A2.shape[0]):
        a = A2[b].T if transA else A2[b]
        bb = B2[b].T if transB else B2[b]
        n, k = a.shape
        m = bb.shape[1]
        c = np.zeros((n, m))
        for i in range(n):
            for j in range(m):
                s = 0.0
                for t in range(k):
                    s += a[i, t] * bb[t, j]
                c[i, j] = s
        outs.append(c)
    return np.stack(outs).reshape(lead + outs[0].shape)


def one_hot_loops(ids, num_classes):
    """src/ops/OneHot.cu:3-14: out[ind] = float(ind % last) == ids[ind / last]."""
    flat = np.asarray(ids, dtype=np.float32).reshape(-1)
    out = np.zeros(flat.size * num_classes, dtype=np.float32)
    for ind in range(out.size):
        out[ind] = 1.0 if np.float32(ind % num_classes) == flat[ind // num_classes] else 0.0
    return out.reshape(np.shape(ids) + (num_classes,))


def embedding_loops(table, ids):
    flat = np.asarray(ids).reshape(-1)
    out = np.empty((flat.size, table.shape[1]), dtype=table.dtype)
    for r in range(flat.size):
        out[r] = table[int(flat[r])]
    return out.reshape(np.shape(ids) + (table.shape[1],))


def embedding_grad_loops(dy, ids, table_shape):
    flat = np.asarray(ids).reshape(-1)
    d2 = dy.reshape(flat.size, table_shape[1]).astype(np.float64)
    g = np.zeros(table_shape, dtype=np.float64)
    for r in range(flat.size):
        g[int(flat[r])] += d2[r]
    return g


def csrmv_loops(data, indptr, indices, nrow, ncol, trans, x):
    """Row-by-row walk of the CSR arrays: y = A x, or y = A^T x (gpu_ops/CuSparse.py:55-58)."""
    y = np.zeros(ncol if trans else nrow, dtype=np.float64)
    for i in range(nrow):
        for j in range(int(indptr[i]), int(indptr[i + 1])):
            if trans:
                y[int(indices[j])] += float(data[j]) * float(x[i])
            else:
                y[i] += float(data[j]) * float(x[int(indices[j])])
    return y


def csrmm_loops(data, indptr, indices, nrow, ncol, transA, B, transB):
    """C = op(A) op(B) entry by entry (gpu_ops/CuSparse.py:150-163)."""
    Bm = np.asarray(B, dtype=np.float64)
    if transB:
        Bm = Bm.T
    n = Bm.shape[1]
    C = np.zeros((ncol if transA else nrow, n), dtype=np.float64)
    for i in range(nrow):
        for j in range(int(indptr[i]), int(indptr[i + 1])):
            c = int(indices[j])
            for t in range(n):
                if transA:
                    C[c, t] += float(data[j]) * Bm[i, t]
                else:
                    C[i, t] += float(data[j]) * Bm[c, t]
    return C
