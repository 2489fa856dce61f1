"""Per-operator timing sweep on one MI355X (the counterpart of the reference's
kernel_profile/*.py sweeps, which time ops one by one through `op.profile`).

    python -m tsplit_amd.opbench [--iters 20] [--filter avg_pool]

Every case launches one operator `iters` times on one stream between two HIP events (after
two untimed launches) and reports the mean launch time with the rate it implies on the
operator's algorithmic work: bytes = every distinct input read once + every output written
once (GB/s against 8000), or 2*M*N*K per matmul (TFLOP/s against 157.3).  Shapes are those
of the ResNet-50 / Inception-v4 / Transformer graphs of the reference's examples.  Prints one
JSON object per case and a final table.
"""
import argparse
import json

import numpy as np

PEAK_GBS = 8000.0
PEAK_TFLOPS = 157.3


def _cases(L, A, E, S):
    """-> list of (name, work, unit, launch) ; A(shape) = random device array, E(shape) = empty one,
    S(nrow, ncol, per_row) = random CSR matrix with per_row entries in every row."""
    c = []

    def add(name, work, unit, fn):
        c.append((name, float(work), unit, fn))

    def n(*shape):
        return int(np.prod(shape))

    # AvgPool: ResNet-50 global pool, Inception-A 3x3 same pool, Inception global pool
    for tag, shp, k, pad, st in (("resnet_global", (64, 2048, 7, 7), 7, 0, 7), ("inception_3x3", (32, 384, 35, 35), 3, 1, 1),
                                 ("inception_3x3_17", (32, 1024, 17, 17), 3, 1, 1), ("inception_global", (32, 1536, 8, 8), 8, 0, 1)):
        oh = (shp[2] + 2 * pad - k) // st + 1
        oshp = (shp[0], shp[1], oh, oh)
        x, y, dy, dx = A(shp), E(oshp), A(oshp), E(shp)
        add("avg_pool_fwd/" + tag, 4 * (n(*shp) + n(*oshp)), "byte",
            lambda s, x=x, y=y, k=k, pad=pad, st=st: L.average_pooling2d(x, k, k, y, pad, st, s))
        add("avg_pool_bwd/" + tag, 4 * (n(*shp) + n(*oshp)), "byte",
            lambda s, dy=dy, dx=dx, k=k, pad=pad, st=st: L.average_pooling2d_gradient(dy, k, k, dx, pad, st, s))
    # MaxPool with overlapping windows: ResNet stem pool, Inception stem pool
    for tag, shp, k, pad, st in (("resnet_3x3s2p1", (64, 64, 112, 112), 3, 1, 2), ("inception_3x3s2", (32, 192, 71, 71), 3, 0, 2)):
        oh = (shp[2] + 2 * pad - k) // st + 1
        oshp = (shp[0], shp[1], oh, oh)
        x, y, dy, dx = A(shp), E(oshp), A(oshp), E(shp)
        add("max_pool_fwd/" + tag, 4 * (n(*shp) + n(*oshp)), "byte",
            lambda s, x=x, y=y, k=k, pad=pad, st=st: L.max_pooling2d(x, k, k, y, pad, st, s))
        add("max_pool_bwd/" + tag, 4 * (2 * n(*shp) + n(*oshp)), "byte",
            lambda s, x=x, dy=dy, dx=dx, k=k, pad=pad, st=st: L.max_pooling2d_gradient(x, dy, k, k, dx, pad, st, s))
    # bias broadcast / bias-gradient reduce
    for tag, rows, cols in (("fc_bias", 64, 1000), ("transformer_bias", 8192, 512), ("transformer_ffn_bias", 8192, 2048)):
        b, out, x = A((cols,)), E((rows, cols)), A((rows, cols))
        add("broadcast_to/" + tag, 4 * (cols + rows * cols), "byte", lambda s, b=b, out=out: L.broadcast_to(b, out, s))
        add("reduce_sum_axis_zero/" + tag, 4 * (cols + rows * cols), "byte",
            lambda s, x=x, b=b: L.reduce_sum_axis_zero(x, b, s))
    for tag, shp in (("resnet_56", (64, 256, 56, 56)), ("resnet_7", (64, 2048, 7, 7)), ("vgg_224", (16, 64, 224, 224))):
        b, out, x = A((shp[1],)), E(shp), A(shp)
        add("conv2d_broadcast_to/" + tag, 4 * (shp[1] + n(*shp)), "byte", lambda s, b=b, out=out: L.conv2d_broadcast_to(b, out, s))
        add("conv2d_reduce_sum/" + tag, 4 * (shp[1] + n(*shp)), "byte", lambda s, x=x, b=b: L.conv2d_reduce_sum(x, b, s))
    # transformer: causal mask broadcast, masked sums, head split/merge, attention matmuls
    tril, mask = A((256, 256)), E((32, 8, 256, 256))
    add("broadcast_shape/causal_mask", 4 * (256 * 256 + n(32, 8, 256, 256)), "byte",
        lambda s: L.broadcast_shape(tril, mask, None, s))
    x3, r01, r2 = A((32, 255, 512)), E((512,)), E((32, 255))
    add("reduce_sum/axes01", 4 * (n(32, 255, 512) + 512), "byte", lambda s: L.reduce_sum(x3, r01, [0, 1], s))
    add("reduce_sum/axis2", 4 * (n(32, 255, 512) + n(32, 255)), "byte", lambda s: L.reduce_sum(x3, r2, [2], s))
    q, qt = A((32, 256, 8, 64)), E((32, 8, 256, 64))
    add("transpose/split_heads_0213", 8 * n(32, 256, 8, 64), "byte", lambda s: L.matrix_transpose(q, qt, [0, 2, 1, 3], s))
    m2, m2t = A((8192, 2048)), E((2048, 8192))
    add("transpose/matrix_8192x2048", 8 * n(8192, 2048), "byte", lambda s: L.matrix_transpose(m2, m2t, [1, 0], s))
    k4, k4t = A((32, 8, 256, 64)), E((32, 8, 64, 256))
    add("transpose/swap_last_two", 8 * n(32, 8, 256, 64), "byte", lambda s: L.matrix_transpose(k4, k4t, [0, 1, 3, 2], s))
    qh, kh, sc = A((32, 8, 256, 64)), A((32, 8, 256, 64)), E((32, 8, 256, 256))
    nb = 32 * 8
    add("batch_matmul/qk_t", 2.0 * nb * 256 * 256 * 64, "flop", lambda s: L.batch_matrix_multiply(qh, False, kh, True, sc, s))
    pr, vh, ctxo = A((32, 8, 256, 256)), A((32, 8, 256, 64)), E((32, 8, 256, 64))
    dv = E((32, 8, 256, 64))
    add("batch_matmul/pv", 2.0 * nb * 256 * 64 * 256, "flop", lambda s: L.batch_matrix_multiply(pr, False, vh, False, ctxo, s))
    add("batch_matmul/p_t_dctx", 2.0 * nb * 256 * 64 * 256, "flop", lambda s: L.batch_matrix_multiply(pr, True, vh, False, dv, s))
    # plain matrix products: Transformer projections / FFN / vocabulary (forward A B, input gradient A B^T,
    # weight gradient A^T B) and the batch-64 fully-connected layers of VGG-16
    for tag, m, k, nn in (("proj_8192x512x512", 8192, 512, 512), ("ffn_8192x512x2048", 8192, 512, 2048),
                          ("vocab_8160x512x32000", 8160, 512, 32000), ("vgg_fc1_64x25088x4096", 64, 25088, 4096),
                          ("vgg_fc2_64x4096x4096", 64, 4096, 4096)):
        ma, mb, mc = A((m, k)), A((k, nn)), A((m, nn))
        da, db = E((m, k)), E((k, nn))
        fl = 2.0 * m * nn * k
        add("matmul/" + tag + "/A_B", fl, "flop",
            lambda s, ma=ma, mb=mb, mc=mc: L.matrix_multiply(ma, False, mb, False, mc, s))
        add("matmul/" + tag + "/dY_Bt", fl, "flop",
            lambda s, mc=mc, mb=mb, da=da: L.matrix_multiply(mc, False, mb, True, da, s))
        add("matmul/" + tag + "/At_dY", fl, "flop",
            lambda s, ma=ma, mc=mc, db=db: L.matrix_multiply(ma, True, mc, False, db, s))
    # pad (Inception-style spatial padding), one-hot labels, where, embedding
    xp, yp = A((32, 96, 35, 35)), E((32, 96, 37, 37))
    add("pad/35_to_37", 4 * (n(32, 96, 35, 35) + n(32, 96, 37, 37)), "byte",
        lambda s: L.pad(xp, yp, [(1, 1), (1, 1)], "CONSTANT", 0.0, s))
    add("pad_gradient/37_to_35", 4 * (n(32, 96, 35, 35) + n(32, 96, 37, 37)), "byte",
        lambda s: L.pad_gradient(yp, xp, [(1, 1), (1, 1)], "CONSTANT", s))
    ids, oh = A((32, 255), ints=32000), E((32, 255, 32000))
    add("one_hot/labels_32000", 4 * (n(32, 255) + n(32, 255, 32000)), "byte", lambda s: L.one_hot(ids, oh, s))
    cond, wa, wb, wo = A((32, 8, 256, 256), ints=2), A((32, 8, 256, 256)), A((32, 8, 256, 256)), E((32, 8, 256, 256))
    add("where/attention_mask", 16 * n(32, 8, 256, 256), "byte", lambda s: L.where(cond, wa, wb, wo, s))
    table, tid, emb = A((32000, 512)), A((32, 256), ints=32000), E((32, 256, 512))
    add("embedding_lookup/32000x512", 4 * (2 * n(32, 256, 512) + n(32, 256)), "byte",
        lambda s: L.embedding_lookup(table, tid, emb, s))
    gtab = E((32000, 512))
    add("embedding_lookup_gradient/32000x512", 4 * (n(32, 256, 512) + n(32, 256) + 2 * n(32000, 512)), "byte",
        lambda s: L.embedding_lookup_gradient(emb, tid, gtab, s))
    # elementwise math on a transformer activation
    xa, xb, xo = A((32, 256, 2048), positive=True), A((32, 256, 2048), positive=True), E((32, 256, 2048))
    ne = n(32, 256, 2048)
    add("sqrt", 8 * ne, "byte", lambda s: L.matrix_sqrt(xa, xo, s))
    add("rsqrt", 8 * ne, "byte", lambda s: L.matrix_rsqrt(xa, xo, s))
    add("sigmoid", 8 * ne, "byte", lambda s: L.sigmoid(xa, xo, s))
    add("tanh", 8 * ne, "byte", lambda s: L.tanh(xa, xo, s))
    add("opposite", 8 * ne, "byte", lambda s: L.matrix_opposite(xa, xo, s))
    add("div_const", 8 * ne, "byte", lambda s: L.matrix_elementwise_divide_const(2.0, xa, xo, s))
    add("divide", 12 * ne, "byte", lambda s: L.matrix_elementwise_divide(xa, xb, xo, s))
    # dropout on the same activation: 8 B/element of values plus one mask bit
    import ctypes
    rsize, rspace = ctypes.c_int(0), ctypes.c_void_p(0)
    L.CuDNN_Dropout(xa, 0.1, xo, rsize, rspace, 1, None)
    add("dropout_fwd", 8.125 * ne, "byte", lambda s: L.CuDNN_Dropout(xa, 0.1, xo, rsize, rspace, 0, s))
    add("dropout_bwd", 8.125 * ne, "byte", lambda s: L.CuDNN_Dropout_gradient(xa, 0.1, xo, rsize, rspace, s))
    # CSR products on a graph-like matrix: 2^20 rows, 16 entries per row, 64 feature columns
    nr, per, nf = 1 << 20, 16, 64
    sp = S(nr, nr, per)
    xv, yv = A((nr,)), E((nr,))
    bm, cm = A((nr, nf)), E((nr, nf))
    csr_bytes = 8 * nr * per + 4 * (nr + 1)
    add("csrmv/1M_rows_16_per_row", csr_bytes + 8 * nr, "byte", lambda s: L.CuSparse_Csrmv(sp, False, xv, yv, s))
    add("csrmv_trans/1M_rows_16_per_row", csr_bytes + 8 * nr, "byte", lambda s: L.CuSparse_Csrmv(sp, True, xv, yv, s))
    add("csrmm/1M_rows_16_per_row_64_cols", csr_bytes + 8 * nr * nf, "byte",
        lambda s: L.CuSparse_Csrmm(sp, False, bm, False, cm, s))
    add("csrmm_transA/1M_rows_16_per_row_64_cols", csr_bytes + 8 * nr * nf, "byte",
        lambda s: L.CuSparse_Csrmm(sp, True, bm, False, cm, s))
    return c


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--filter", default="")
    a = ap.parse_args()
    from . import gpu_links as L
    from . import ndarray, stream
    from .timing import EventTimer
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    rng = np.random.RandomState(7)

    def A(shape, ints=0, positive=False):
        if ints:
            v = rng.randint(0, ints, size=shape).astype(np.float32)
        elif positive:
            v = (rng.rand(*shape) + 0.5).astype(np.float32)
        else:
            v = rng.standard_normal(size=shape).astype(np.float32)
        return ndarray.array(v, ctx)

    def E(shape):
        return ndarray.empty(shape, ctx)

    def S(nrow, ncol, per_row):
        cols = np.sort(rng.randint(0, ncol, size=(nrow, per_row)), axis=1).astype(np.int32).reshape(-1)
        ptr = (np.arange(nrow + 1, dtype=np.int64) * per_row).astype(np.int32)
        vals = rng.standard_normal(size=nrow * per_row).astype(np.float32)
        d, r, c = ndarray.empty(vals.shape, ctx), ndarray.empty(ptr.shape, ctx), ndarray.empty(cols.shape, ctx)
        d._sync_copyfrom(vals)
        r._sync_copyfrom(ptr, np.int32)
        c._sync_copyfrom(cols, np.int32)
        return ndarray.ND_Sparse_Array(d, r, c, nrow, ncol)

    timer = EventTimer(ctx)
    rows = []
    for name, work, unit, fn in _cases(L, A, E, S):
        if a.filter and a.filter not in name:
            continue
        fn(st)
        fn(st)
        st.sync()
        ea, eb = timer._mk(), timer._mk()
        ea.record(st)
        for _ in range(a.iters):
            fn(st)
        eb.record(st)
        st.sync()
        ms = timer.elapsed_ms(ea, eb) / a.iters
        rate = work / (ms * 1e-3) / (1e12 if unit == "flop" else 1e9)
        peak = PEAK_TFLOPS if unit == "flop" else PEAK_GBS
        row = {"op": name, "us": ms * 1e3, "achieved": rate, "unit": "TFLOP/s" if unit == "flop" else "GB/s",
               "frac": rate / peak}
        rows.append(row)
        print(json.dumps(row), flush=True)
    print("\n%-44s %10s %12s %8s" % ("operator/case", "us", "rate", "of peak"))
    for r in rows:
        print("%-44s %10.1f %8.1f %-7s %6.1f%%" % (r["op"], r["us"], r["achieved"], r["unit"], 100 * r["frac"]))


if __name__ == "__main__":
    main()
