"""The 3x3 / stride 1 / pad 1 layers of VGG-16 one by one on one MI355X: every pass on the direct kernels
and through the Winograd routine, with the time and rate of the GEMM launch inside the routine.

    python -m tsplit_amd.winobench [--iters 10] [--split-bf16]

Shapes are those of the benchmark step (batch 64; the 224x224 and 112x112 layers as micro-tensors of 16
images).  A call is timed over `iters` back-to-back launches between two HIP events after two untimed
ones; the GEMM inside a Winograd call by the library's own event pairs (TSplit_WinogradGemmTiming).
"direct-equivalent" rates count the direct algorithm's FLOP, of which the routine executes a quarter;
GEMM rates count executed FLOP (2 * 36 * rows * tiles * depth) against the 157.3 TFLOP/s fp32 matrix peak.
With --split-bf16 the GEMMs of layers with more than 64 channels on both sides take their products as six
bf16 x bf16 terms (TSplit_SplitBf16); their rate is then the fp32-equivalent one (the same FLOP count).
Layers with 64 channels on one side run forward and data gradient as one kernel (transforms inside): its "GEMM" time
is the whole call's.
Prints one JSON object per layer and pass and a final table.
"""
import argparse
import json
import os

import numpy as np

LAYERS = [(16, 64, 64, 224), (16, 64, 128, 112), (16, 128, 128, 112), (64, 128, 256, 56), (64, 256, 256, 56),
          (64, 256, 512, 28), (64, 512, 512, 28), (64, 512, 512, 14)]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--split-bf16", action="store_true")
    ap.add_argument("--layers", type=int, default=len(LAYERS), help="only the first so many layers")
    a = ap.parse_args()
    from . import gpu_links as L, ndarray, stream
    from .timing import EventTimer
    ctx = ndarray.gpu(0)
    L.split_bf16(a.split_bf16)
    st = stream.create_stream_handle(ctx)
    timer = EventTimer(ctx)
    rng = np.random.RandomState(0)
    rows = []
    for n, c, o, hw in LAYERS[:a.layers]:
        x = ndarray.array(rng.standard_normal((n, c, hw, hw)).astype(np.float32), ctx)
        w = ndarray.array((rng.standard_normal((o, c, 3, 3)) / np.sqrt(9.0 * c)).astype(np.float32), ctx)
        dy = ndarray.array(rng.standard_normal((n, o, hw, hw)).astype(np.float32), ctx)
        y, dx, dw = ndarray.empty((n, o, hw, hw), ctx), ndarray.empty((n, c, hw, hw), ctx), ndarray.empty((o, c, 3, 3), ctx)
        calls = (("forward", lambda: L.CuDNN_conv2d(x, w, y, 1, 1, 1, st), 0, o, c),
                 ("data gradient", lambda: L.CuDNN_conv2d_gradient_of_data(w, dy, dx, 1, 1, 1, st), 0, c, o),
                 ("filter gradient", lambda: L.CuDNN_conv2d_gradient_of_filter(x, dy, dw, 1, 1, 1, st), 1, o, c))
        flop = 2.0 * n * o * hw * hw * c * 9
        for name, fn, kind, gemm_rows, depth in calls:
            row = {"images": n, "in_channels": c, "out_channels": o, "plane": hw, "pass": name}
            for forced, tag in (("0", "direct"), ("1", "winograd")):
                os.environ["TSPLIT_CONV_WINOGRAD"] = forced
                fn()
                fn()
                st.sync()
                ea, eb = timer._mk(), timer._mk()
                ea.record(st)
                for _ in range(a.iters):
                    fn()
                eb.record(st)
                st.sync()
                us = timer.elapsed_ms(ea, eb) / a.iters * 1e3
                row[tag + "_us"] = us
                row[tag + "_tflops_direct_equivalent"] = flop / us / 1e6
            # the GEMM inside the Winograd call, by the library's event pairs
            L.winograd_gemm_timing(True)
            for _ in range(a.iters):
                fn()
            st.sync()
            launches = ms = gf = 0
            for k in ((1, 4, 6) if kind == 1 else (0, 2, 3, 5)):
                ln, m, f, _ = L.winograd_gemm_times(kind=k)
                launches, ms, gf = launches + ln, ms + m, gf + f
            L.winograd_gemm_timing(False)
            row["gemm_us"] = ms / launches * 1e3
            row["gemm_tflops_executed"] = gf / (ms * 1e-3) / 1e12
            row["gemm_frac_of_matrix_peak"] = row["gemm_tflops_executed"] / 157.3
            rows.append(row)
            print(json.dumps(row), flush=True)
        os.environ.pop("TSPLIT_CONV_WINOGRAD", None)
    print("\n%-26s %-16s %10s %10s %9s %9s %10s %8s" % ("layer (images C->O @ plane)", "pass", "direct us", "winograd us", "direct TF", "wino TF*",
                                                         "GEMM us", "GEMM TF"))
    for r in rows:
        print("%-26s %-16s %10.1f %10.1f %9.1f %9.1f %10.1f %8.1f" % (
            "%d x %d->%d @ %d" % (r["images"], r["in_channels"], r["out_channels"], r["plane"]), r["pass"], r["direct_us"],
            r["winograd_us"], r["direct_tflops_direct_equivalent"], r["winograd_tflops_direct_equivalent"], r["gemm_us"],
            r["gemm_tflops_executed"]))
    print("(* rate of the direct algorithm's FLOP count)")
    if a.split_bf16:
        print("(split-bf16 products in the GEMMs of layers with more than 64 channels on both sides: GEMM TF is the "
              "fp32-equivalent rate)")


if __name__ == "__main__":
    main()
