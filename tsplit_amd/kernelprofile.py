"""One operator at a time, GPU next to CPU: the counterpart of the reference's kernel_profile/ scripts
(kernel_profile/conv2d.py:49-52,91, bn.py:33-49, relu.py:12-25, matmul.py:34-60, maxpool.py), which time one
operator through `op.profile` (the ProfilerHandle of the C ABI) over a sweep of batch sizes.

    python -m tsplit_amd.kernelprofile [--batches 1,16,64] [--repeat 10] [--no-cpu]

Shapes are the reference's: convolution [B,64,224,224] * [128,64,3,3] pad 1 and [B,64,32,32] * [128,64,3,3]
(forward, data gradient, filter gradient), BatchNorm and Relu on [B,64,224,224], the product [B,1024] x
[1024,1024] and [100,4096] x [4096,4096], and 2x2 / stride 2 max pooling on [B,64,224,224].

GPU: every call is made with a ProfilerHandle, as the reference's `profile` methods make it: the library
brackets the operator with events on its stream, waits, and writes the milliseconds into the struct; the mean
of `repeat` calls after one untimed call.  CPU: the same operator on the same shape through PyTorch-CPU's
bundled oneDNN (the stand-in for the reference's dnnl operators, which cannot be compiled against the oneDNN
on this machine), all host cores, the mean of 3 calls after one.  Rates are on algorithmic work: 2 x
multiply-adds against 157.3 TFLOP/s, or bytes of every operand read once and every result written once
against 8 TB/s.  One JSON object per case, then a table."""
import argparse
import json
import os
import time

import numpy as np

PEAK_TFLOPS, PEAK_GBS = 157.3, 8000.0


def _cpu_ms(fn, repeat=3):
    fn()
    t0 = time.perf_counter()
    for _ in range(repeat):
        fn()
    return (time.perf_counter() - t0) / repeat * 1e3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batches", default="1,16,64")
    ap.add_argument("--repeat", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true")
    a = ap.parse_args()
    from . import gpu_links as L, ndarray, profiler, stream
    ctx = ndarray.gpu(0)
    st = stream.create_stream_handle(ctx)
    prof = profiler.CreateProfiler()
    rng = np.random.RandomState(123)
    torch = F = None
    if not a.no_cpu:
        try:
            import torch
            import torch.nn.functional as F
            torch.set_num_threads(os.cpu_count() or 1)
        except Exception:
            torch = None

    def gpu_ms(call):
        call()
        total = 0.0
        for _ in range(a.repeat):
            call()
            total += prof.time
        return total / a.repeat

    rows = []

    def case(name, batch, work, unit, gpu_call, cpu_call):
        ms = gpu_ms(gpu_call)
        rate = work / (ms * 1e-3) / (1e12 if unit == "flop" else 1e9)
        row = {"op": name, "batch": batch, "gpu_ms": ms, "achieved": rate, "unit": "TFLOP/s" if unit == "flop" else "GB/s",
               "frac": rate / (PEAK_TFLOPS if unit == "flop" else PEAK_GBS)}
        if torch is not None and cpu_call is not None:
            with torch.no_grad():
                row["cpu_ms"] = _cpu_ms(cpu_call)
            row["cpu_cores"] = int(torch.get_num_threads())
            row["speedup"] = row["cpu_ms"] / ms
        rows.append(row)
        print(json.dumps(row), flush=True)

    def dev(v):
        return ndarray.array(v, ctx)

    for B in [int(v) for v in a.batches.split(",")]:
        for hw in (224, 32):
            x = rng.normal(scale=0.1, size=(B, 64, hw, hw)).astype(np.float32)
            w = rng.normal(scale=0.1, size=(128, 64, 3, 3)).astype(np.float32)
            dy = rng.normal(scale=0.1, size=(B, 128, hw, hw)).astype(np.float32)
            gx, gw, gdy = dev(x), dev(w), dev(dy)
            y, dx, dw = ndarray.empty(dy.shape, ctx), ndarray.empty(x.shape, ctx), ndarray.empty(w.shape, ctx)
            flop = 2.0 * B * 128 * hw * hw * 64 * 9
            tx, tw, tdy = (torch.from_numpy(v) for v in (x, w, dy)) if torch is not None else (None, None, None)
            tag = "conv %dx%d 64->128" % (hw, hw)
            case(tag + " forward", B, flop, "flop", lambda: L.CuDNN_conv2d(gx, gw, y, 1, 1, 1, st, prof),
                 (lambda: F.conv2d(tx, tw, padding=1)) if torch is not None else None)
            case(tag + " data gradient", B, flop, "flop", lambda: L.CuDNN_conv2d_gradient_of_data(gw, gdy, dx, 1, 1, 1, st, prof),
                 (lambda: torch.nn.grad.conv2d_input(tx.shape, tw, tdy, padding=1)) if torch is not None else None)
            case(tag + " filter gradient", B, flop, "flop", lambda: L.CuDNN_conv2d_gradient_of_filter(gx, gdy, dw, 1, 1, 1, st, prof),
                 (lambda: torch.nn.grad.conv2d_weight(tx, tw.shape, tdy, padding=1)) if torch is not None else None)
            del gx, gw, gdy, y, dx, dw
        x = rng.normal(scale=0.1, size=(B, 64, 224, 224)).astype(np.float32)
        g = rng.normal(scale=0.1, size=(1, 64, 1, 1)).astype(np.float32)
        b = rng.normal(scale=0.1, size=(1, 64, 1, 1)).astype(np.float32)
        gx, gg, gb, out = dev(x), dev(g), dev(b), ndarray.empty(x.shape, ctx)
        up = rng.normal(scale=0.1, size=x.shape).astype(np.float32)            # the gradient arriving from above
        gup = dev(up)
        tup = torch.from_numpy(up) if torch is not None else None
        dg, db = ndarray.empty(g.shape, ctx), ndarray.empty(g.shape, ctx)
        n = float(x.size)
        tx = torch.from_numpy(x) if torch is not None else None
        tg, tb = (torch.from_numpy(g.reshape(-1)), torch.from_numpy(b.reshape(-1))) if torch is not None else (None, None)
        if torch is not None:
            _, tmean, tistd = torch.ops.aten.native_batch_norm(tx, tg, tb, None, None, True, 0.1, 0.01)
        case("batchnorm 224x224x64 forward", B, 8 * n, "byte",
             lambda: L.CuDNN_Batch_Normalization(gx, gg, gb, out, None, None, 0.99, 0.01, st, prof),
             (lambda: F.batch_norm(tx, None, None, tg, tb, training=True, eps=0.01)) if torch is not None else None)
        case("batchnorm 224x224x64 gradient", B, 12 * n, "byte",
             lambda: L.CuDNN_Batch_Normalization_gradient(gup, gx, gg, out, dg, db, None, None, 0.01, st, prof),
             (lambda: torch.ops.aten.native_batch_norm_backward(tup, tx, tg, None, None, tmean, tistd, True, 0.01, [True, True, True]))
             if torch is not None else None)
        case("relu 224x224x64 forward", B, 8 * n, "byte", lambda: L.relu(gx, out, st, prof),
             (lambda: F.relu(tx)) if torch is not None else None)
        case("relu 224x224x64 gradient", B, 12 * n, "byte", lambda: L.relu_gradient(gx, gup, out, st, prof),
             (lambda: torch.ops.aten.threshold_backward(tup, tx, 0.0)) if torch is not None else None)
        pooled = ndarray.empty((B, 64, 112, 112), ctx)
        pup = rng.normal(scale=0.1, size=(B, 64, 112, 112)).astype(np.float32)
        gpup = dev(pup)
        if torch is not None:
            tpup = torch.from_numpy(pup)
            _, tidx = F.max_pool2d(tx, 2, 2, return_indices=True)
        case("maxpool 2x2/2 224x224x64 forward", B, 4 * (n + n / 4), "byte", lambda: L.CuDNN_max_pooling2d(gx, 2, 2, pooled, 0, 2, st, prof),
             (lambda: F.max_pool2d(tx, 2, 2)) if torch is not None else None)
        case("maxpool 2x2/2 224x224x64 gradient", B, 4 * (2 * n + n / 4), "byte",
             lambda: L.CuDNN_max_pooling2d_gradient(pooled, gpup, gx, 2, 2, out, 0, 2, st, prof),
             (lambda: torch.ops.aten.max_pool2d_with_indices_backward(tpup, tx, [2, 2], [2, 2], [0, 0], [1, 1], False, tidx))
             if torch is not None else None)
        del gx, out, pooled, gup, gpup
        for rows_, k, cols in ((B, 1024, 1024), (100, 4096, 4096)):
            if rows_ == 100 and B != int(a.batches.split(",")[0]):
                continue
            m1 = rng.normal(scale=0.1, size=(rows_, k)).astype(np.float32)
            m2 = rng.normal(scale=0.1, size=(k, cols)).astype(np.float32)
            ga, gb2, gc = dev(m1), dev(m2), ndarray.empty((rows_, cols), ctx)
            ta, tb2 = (torch.from_numpy(m1), torch.from_numpy(m2)) if torch is not None else (None, None)
            case("matmul [%d,%d] x [%d,%d]" % (rows_, k, k, cols), rows_, 2.0 * rows_ * k * cols, "flop",
                 lambda: L.matrix_multiply(ga, False, gb2, False, gc, st, prof),
                 (lambda: torch.mm(ta, tb2)) if torch is not None else None)
    print("\n%-40s %6s %10s %16s %8s %10s %9s" % ("operator", "batch", "GPU ms", "rate", "of peak", "CPU ms", "GPU/CPU"))
    for r in rows:
        print("%-40s %6d %10.3f %9.1f %-7s %7.1f%% %10s %9s" % (r["op"], r["batch"], r["gpu_ms"], r["achieved"], r["unit"], 100 * r["frac"],
                                                               "%.1f" % r["cpu_ms"] if "cpu_ms" in r else "-",
                                                               "%.0fx" % r["speedup"] if "speedup" in r else "-"))
    print("conv rates count the direct algorithm's FLOP (2 * B * O * H * W * C * 9); layers the Winograd routine takes execute a quarter of "
          "them, so such a call can read above 100 % of the matrix peak.  BatchNorm forward on a tensor no convolution of this library has "
          "just written reads it twice (statistics, then apply): 12 B per element moved for the 8 counted.")
    if rows and "cpu_cores" in rows[0]:
        print("CPU: PyTorch %s (bundled oneDNN), %d threads" % (torch.__version__, rows[0]["cpu_cores"]))


if __name__ == "__main__":
    main()
