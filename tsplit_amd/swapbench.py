"""Copy rates of the swap path on one MI355X box: pinned host pool <-> HBM through
DLArrayCopyFromTo on a copy stream, alone and while a convolution runs on the compute stream.

    python -m tsplit_amd.swapbench [--mb 1024]

Prints one JSON object.  Times come from HIP events on the stream each operation runs on.
"""
import argparse
import json

import numpy as np


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--mb", type=int, default=1024)
    a = ap.parse_args()
    from . import gpu_links as L
    from . import ndarray, stream
    from .timing import EventTimer
    ctx = ndarray.gpu(0)
    compute, copy = stream.create_stream_handle(ctx), stream.create_stream_handle(ctx)
    timer = EventTimer(ctx)
    n = a.mb * (1 << 20) // 4
    dev = ndarray.empty((n,), ctx)
    L.array_set(dev, 1.0, compute)
    compute.sync()
    host = ndarray.empty((n,), ndarray.cpu(0))
    rng = np.random.RandomState(0)
    x = ndarray.array(rng.standard_normal((64, 256, 56, 56)).astype(np.float32), ctx)
    w = ndarray.array((rng.standard_normal((256, 256, 3, 3)) * 0.02).astype(np.float32), ctx)
    y = ndarray.empty((64, 256, 56, 56), ctx)

    def timed(stream_, fn, reps):
        fn()
        stream_.sync()
        ea, eb = timer._mk(), timer._mk()
        ea.record(stream_)
        for _ in range(reps):
            fn()
        eb.record(stream_)
        stream_.sync()
        return timer.elapsed_ms(ea, eb) / reps

    gb = a.mb / 1024.0 * 1.073741824
    d2h = timed(copy, lambda: host.async_d2h(dev, copy), 3)
    h2d = timed(copy, lambda: dev.async_h2d(host, copy), 3)
    conv = timed(compute, lambda: L.CuDNN_conv2d(x, w, y, 1, 1, 1, compute), 10)
    # both at once: enough convolutions to cover one swap-out plus one swap-in
    reps = max(1, int((d2h + h2d) / conv) + 1)
    ea, eb, ca, cb = timer._mk(), timer._mk(), timer._mk(), timer._mk()
    ea.record(compute)
    ca.record(copy)
    host.async_d2h(dev, copy)
    dev.async_h2d(host, copy)
    cb.record(copy)
    for _ in range(reps):
        L.CuDNN_conv2d(x, w, y, 1, 1, 1, compute)
    eb.record(compute)
    compute.sync()
    copy.sync()
    conv_with = timer.elapsed_ms(ea, eb) / reps
    copy_with = timer.elapsed_ms(ca, cb)
    print(json.dumps({
        "buffer_MiB": a.mb, "d2h_GBps": gb / (d2h * 1e-3), "h2d_GBps": gb / (h2d * 1e-3),
        "conv_ms_alone": conv, "conv_ms_during_copies": conv_with,
        "d2h_plus_h2d_ms_alone": d2h + h2d, "d2h_plus_h2d_ms_during_conv": copy_with,
        "conv_slowdown": conv_with / conv, "copy_slowdown": copy_with / (d2h + h2d)}))


if __name__ == "__main__":
    main()
