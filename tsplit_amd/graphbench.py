"""Times one training step (forward, backward, SGD) of the branched example networks at the
sizes of the reference's benchmark configurations, on one MI355X through the C ABI.

    python -m tsplit_amd.graphbench --net resnet50|resnet101|inception_v4|transformer|lstm|mlp|vgg19 [--steps 5] [--warmup 2] [--record] [--split-bf16]

--split-bf16 turns on the opt-in split-bf16 products of the matrix products and the Winograd GEMMs
(TSplit_SplitBf16).  --record issues the step once into a HIP graph after the warm-up and times replays of that graph
(one host call per step) instead of Python issuing every operator again.

Prints one JSON object: samples/s, ms/step, final loss, operator calls per step, and - from a second pass
of the same steps in which every primitive call is bracketed by HIP events on the compute stream (--no-kernels
skips it) - `kernels`: per operator class the calls and milliseconds per step and the rate on algorithmic work
(2 x multiply-adds for contractions against the fp32 matrix peak of 157.3 TFLOP/s; bytes of each distinct operand
read once and each result written once for the rest, against 8 TB/s), and `roofline`: the class with the largest
share of the step.  Synthetic seeded inputs; parameters as in workloads.py.  (The headline benchmark of this repository is
bench.py; this sweep only shows the other configurations running at their real shapes.)
"""
import argparse
import json
import time

import numpy as np

PEAK_TFLOPS_FP32_MFMA = 157.3
PEAK_HBM_GBS = 8000.0


def _n(shape):
    n = 1
    for v in shape:
        n *= int(v)
    return float(n)


def _pooled(xs, k, pad, s):
    return (xs[0], xs[1], (xs[2] + 2 * pad - k) // s + 1, (xs[3] + 2 * pad - k) // s + 1)


# primitive of graph.GpuBackend -> (operator class, algorithmic work, "flop" | "byte") from the call's arguments
WORK = {
    "conv2d": lambda x, w, xs, ws, ph, pw, s: ("conv_fwd", 2.0 * xs[0] * ws[0] * ((xs[2] + 2 * ph - ws[2]) // s + 1)
                                                * ((xs[3] + 2 * pw - ws[3]) // s + 1) * ws[1] * ws[2] * ws[3], "flop"),
    "conv2d_grad_data": lambda w, dy, xs, ph, pw, s: ("conv_bwd_data", 2.0 * _n(dy.shape) * _n(w.shape[1:]), "flop"),
    "conv2d_grad_filter": lambda x, dy, ws, ph, pw, s: ("conv_bwd_filter", 2.0 * _n(dy.shape) * _n(ws[1:]), "flop"),
    "matmul": lambda a, ta, b, tb, out: ("matmul", 2.0 * _n(out) * (a.shape[0] if ta else a.shape[1]), "flop"),
    "batch_matmul": lambda a, ta, b, tb, out: ("batch_matmul", 2.0 * _n(out) * (a.shape[-2] if ta else a.shape[-1]), "flop"),
    "bn": lambda x, g, b, xs, eps: ("bn_fwd", 8.0 * _n(xs), "byte"),
    "bn_grad": lambda dy, x, g, xs, eps: ("bn_bwd", 12.0 * _n(xs), "byte"),
    "bn_relu": lambda x, g, b, xs, eps: ("bn_relu_fwd", 8.0 * _n(xs), "byte"),
    "bn_relu_grad": lambda dy, x, g, b, m, i, xs, eps: ("bn_relu_bwd", 12.0 * _n(xs), "byte"),
    "relu": lambda x, shape: ("relu_fwd", 8.0 * _n(shape), "byte"),
    "relu_grad": lambda x, dy, shape: ("relu_bwd", 12.0 * _n(shape), "byte"),
    "max_pool": lambda x, xs, k, pad, s: ("maxpool_fwd", 4.0 * (_n(xs) + _n(_pooled(xs, k, pad, s))), "byte"),
    "max_pool_grad": lambda x, y, dy, xs, k, pad, s: ("maxpool_bwd", 4.0 * (2 * _n(xs) + _n(dy.shape)), "byte"),
    "avg_pool": lambda x, xs, k, pad, s: ("avgpool_fwd", 4.0 * (_n(xs) + _n(_pooled(xs, k, pad, s))), "byte"),
    "avg_pool_grad": lambda x, y, dy, xs, k, pad, s: ("avgpool_bwd", 4.0 * (_n(xs) + _n(dy.shape)), "byte"),
    "add": lambda a, b, shape: ("add", 12.0 * _n(shape), "byte"),
    "mul": lambda a, b, shape: ("mul", 12.0 * _n(shape), "byte"),
    "mul_const": lambda a, c, shape: ("mul_const", 8.0 * _n(shape), "byte"),
    "add_const": lambda a, c, shape: ("add_const", 8.0 * _n(shape), "byte"),
    "sigmoid": lambda x, shape: ("sigmoid", 8.0 * _n(shape), "byte"),
    "tanh": lambda x, shape: ("tanh", 8.0 * _n(shape), "byte"),
    "slice": lambda x, begin, out: ("slice", 8.0 * _n(out), "byte"),
    "slice_grad": lambda dy, begin, ins: ("slice_grad", 4.0 * (_n(dy.shape) + _n(ins)), "byte"),
    "broadcast_shape": lambda x, out: ("broadcast", 4.0 * (_n(x.shape) + _n(out)), "byte"),
    "broadcast_to": lambda x, out: ("broadcast", 4.0 * (_n(x.shape) + _n(out)), "byte"),
    "reduce_sum": lambda x, axes, out: ("reduce_sum", 4.0 * (_n(x.shape) + _n(out)), "byte"),
    "reduce_sum_axis_zero": lambda x, out: ("reduce_sum", 4.0 * (_n(x.shape) + _n(out)), "byte"),
    "concat": lambda a, b, out, axis: ("concat", 8.0 * _n(out), "byte"),
    "concat_grad": lambda dout, ins, axis, idx: ("concat_grad", 8.0 * _n(ins), "byte"),
    "transpose": lambda x, perm, out: ("transpose", 8.0 * _n(out), "byte"),
    "reshape": lambda x, shape: ("reshape_copy", 8.0 * _n(shape), "byte"),
    "where": lambda c, a, b, shape: ("where", 16.0 * _n(shape), "byte"),
    "one_hot": lambda ids, out: ("one_hot", 4.0 * (_n(ids.shape) + _n(out)), "byte"),
    "embedding": lambda table, ids, out: ("embedding", 4.0 * (_n(ids.shape) + 2 * _n(out)), "byte"),
    "embedding_grad": lambda dy, ids, ts: ("embedding_grad", 4.0 * (_n(dy.shape) + 2 * _n(ts)), "byte"),
    "zeros": lambda shape: ("set", 4.0 * _n(shape), "byte"),
    "softmax_ce": lambda logits, labels: ("softmax_ce_fwd", 8.0 * _n(logits.shape), "byte"),
    "softmax_ce_grad": lambda logits, labels, shape, seed=1.0: ("softmax_ce_grad", 12.0 * _n(shape), "byte"),
    "sgd": lambda p, g, lr: ("sgd", 12.0 * _n(p.shape), "byte"),
}


def timed_backend(backend, timer):
    """Wraps every primitive of `backend` listed in WORK so that, while `timer.enabled`, the call is bracketed
    by events on the compute stream and booked under its operator class with its algorithmic work."""
    for name, work in WORK.items():
        fn = getattr(backend, name)

        def wrapped(*args, _fn=fn, _work=work, **kwargs):
            if not timer.enabled:
                return _fn(*args, **kwargs)
            tag, amount, unit = _work(*args, **kwargs)
            timer.begin(backend.stream)
            out = _fn(*args, **kwargs)
            timer.end(backend.stream, tag, amount, unit)
            return out
        setattr(backend, name, wrapped)
    return backend


def kernel_table(timer, steps):
    """-> (kernels dict sorted by time, roofline dict of the largest class)"""
    k = timer.collect()
    kernels = {}
    for tag, d in sorted(k.items(), key=lambda kv: -kv[1]["ms_total"]):
        peak = PEAK_TFLOPS_FP32_MFMA if d["unit"] == "flop" else PEAK_HBM_GBS
        kernels[tag] = {"calls_per_step": d["calls"] / steps, "ms_per_step": d["ms_total"] / steps, "ms_avg": d["ms_avg"],
                        "achieved": d["rate"], "unit": "TFLOP/s" if d["unit"] == "flop" else "GB/s", "frac": d["rate"] / peak}
    dom = next(iter(kernels))
    dd = k[dom]
    peak = PEAK_TFLOPS_FP32_MFMA if dd["unit"] == "flop" else PEAK_HBM_GBS
    roofline = {"kernel": dom, "bound": "mfma" if dd["unit"] == "flop" else "hbm", "achieved": dd["rate"], "peak": peak,
                "unit": "TFLOP/s" if dd["unit"] == "flop" else "GB/s", "frac": dd["rate"] / peak, "traffic": None,
                "per_launch": dd["work_per_call"], "ms_avg": dd["ms_avg"],
                "note": "an operator class (all shapes of the step together), one event pair per call"}
    return kernels, roofline


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--net", default="resnet50", choices=["resnet50", "resnet101", "inception_v4", "transformer", "lstm", "mlp", "vgg19"])
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--lr", type=float, default=1e-4)
    ap.add_argument("--record", action="store_true", help="record the step into a graph and time its replays")
    ap.add_argument("--split-bf16", action="store_true")
    ap.add_argument("--fused", action="store_true",
                    help="BatchNorm + Relu pairs of the conv nets as one node each (TSplit_BatchNormRelu / _gradient)")
    ap.add_argument("--no-kernels", action="store_true", help="skip the second, per-call instrumented pass")
    a = ap.parse_args()
    from . import gpu_links, graph, ndarray, stream, workloads
    ctx = ndarray.gpu(0)
    gpu_links.split_bf16(a.split_bf16)
    if a.net in ("mlp", "vgg19"):
        return layer_list(a, ctx)
    st = stream.create_stream_handle(ctx)
    from .timing import EventTimer
    timer = EventTimer(ctx, chained=True)
    backend = timed_backend(graph.GpuBackend(ctx, st), timer)
    rng = np.random.RandomState(123)
    store = workloads.ParamStore(123)
    calls = [0]

    if a.net in ("resnet50", "resnet101"):
        n = a.batch or 64
        stages = (3, 4, 6, 3) if a.net == "resnet50" else (3, 4, 23, 3)
        x = rng.standard_normal((n, 3, 224, 224)).astype(np.float32)
        y = np.zeros((n, 1000), np.float32)
        y[np.arange(n), rng.randint(0, 1000, n)] = 1

        def build(t, b, cache):
            return workloads.resnet(t, b, cache["x"], cache["y"], blocks=stages)
        inputs = {"x": x, "y": y}
        desc = "ResNet-%s, fp32 NCHW, batch %d, 3x224x224, 1000 classes" % (a.net[6:], n)
    elif a.net == "inception_v4":
        n = a.batch or 32
        x = rng.standard_normal((n, 3, 299, 299)).astype(np.float32)
        y = np.zeros((n, 1000), np.float32)
        y[np.arange(n), rng.randint(0, 1000, n)] = 1

        def build(t, b, cache):
            return workloads.inception_v4(t, b, cache["x"], cache["y"])
        inputs = {"x": x, "y": y}
        desc = "Inception-v4, fp32 NCHW, batch %d, 3x299x299, 1000 classes" % n
    elif a.net == "lstm":
        n = a.batch or 512
        x = rng.uniform(0, 1, size=(n, 28 * 28)).astype(np.float32)
        y = np.zeros((n, 10), np.float32)
        y[np.arange(n), rng.randint(0, 10, n)] = 1

        def build(t, b, cache):
            return workloads.lstm(t, b, cache["x"], cache["y"])
        inputs = {"x": x, "y": y}
        desc = "LSTM classifier, 28 frames x 28 values, 128 hidden units, 10 classes, batch %d" % n
    else:
        n = a.batch or 32
        # no softmax in this graph: masked scores are set to 0 and values are kept small so that twelve
        # blocks stay finite
        cfg = workloads.TransformerConfig(batch=n, mask_value=0.0, embed_std=0.0002, pos_amplitude=0.003)
        inputs = {"xs": rng.randint(1, cfg.vocab, size=(n, cfg.len1)).astype(np.float32),
                  "yi": rng.randint(1, cfg.vocab, size=(n, cfg.len2)).astype(np.float32),
                  "yo": rng.randint(1, cfg.vocab, size=(n, cfg.len2)).astype(np.float32)}

        def build(t, b, cache):
            return workloads.transformer(t, b, cfg, cache["xs"], cache["yi"], cache["yo"])
        desc = "Transformer 6+6 blocks, d_model 512, 8 heads, FFN 2048, length 256, batch %d, vocab 32000" % n

    binder = None
    dev_inputs = None
    loss_val = float("nan")

    def one_step():
        nonlocal binder, dev_inputs
        t = graph.Tape(backend)
        t.fuse_bn_relu = a.fused
        if binder is None:
            binder = workloads.Binder(t, store)
            dev_inputs = {k: binder.input(v) for k, v in inputs.items()}      # resident before timing
        else:
            binder.t, binder._n = t, 0
            for v in binder.vars.values():
                v.grad = None
        loss, _ = build(t, binder, dev_inputs)
        calls[0] = len(t._nodes)
        t.backward(loss)
        binder.sgd_step(a.lr)
        return loss

    for _ in range(a.warmup):
        one_step()
    backend.sync()
    if a.record:
        with stream.recording(st) as rec:
            loss = one_step()
        rec.graph.launch(st)            # first launch uploads the graph
        backend.sync()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            rec.graph.launch(st)
        backend.sync()
        dt = time.perf_counter() - t0
    else:
        t0 = time.perf_counter()
        for _ in range(a.steps):
            loss = one_step()
        backend.sync()
        dt = time.perf_counter() - t0
    loss_val = float(loss.value.asnumpy()[0])
    out = {"net": a.net, "workload": desc, "samples_per_s": n * a.steps / dt, "ms_per_step": dt / a.steps * 1e3,
           "steps": a.steps, "warmup": a.warmup, "final_loss": loss_val, "forward_ops_per_step": calls[0], "recorded": bool(a.record),
           "fused_bn_relu": bool(a.fused), "dtype": "f32", "data": "synthetic"}
    if not a.no_kernels and not a.record:
        timer.enabled = True
        t1 = time.perf_counter()
        for _ in range(a.steps):
            one_step()
        backend.sync()
        out["instrumented_ms_per_step"] = (time.perf_counter() - t1) / a.steps * 1e3
        timer.enabled = False
        out["kernels"], out["roofline"] = kernel_table(timer, a.steps)
        conv = [v for k, v in out["kernels"].items() if k.startswith("conv_")]
        if conv:
            ms = sum(v["ms_per_step"] for v in conv)
            out["conv_mfma_util_pct"] = 100.0 * sum(v["achieved"] * v["ms_per_step"] for v in conv) / ms / PEAK_TFLOPS_FP32_MFMA
    print(json.dumps(out))


def layer_list(a, ctx):
    """Nets that are plain layer lists, on the layer-list trainer: the 784-256-256-10 MLP of the smallest
    benchmark configuration (batch 128, SGD 0.1; 13 launches per step, so the step is the host's launch
    rate unless recorded) and VGG-19 (batch 64, momentum SGD, as bench.py runs VGG-16)."""
    from . import ndarray, trainer
    rng = np.random.RandomState(123)
    if a.net == "mlp":
        n, classes = a.batch or 128, 10
        spec, opt = trainer.mlp_spec(), ("sgd", 0.1)
        x = rng.uniform(0, 1, size=(n, 784)).astype(np.float32)
        desc = "MLP 784-256-256-10, batch %d, SGD" % n
    else:
        n, classes = a.batch or 64, 1000
        spec, opt = trainer.vgg19_spec(1000, 224), ("momentum", 1e-4, 0.9)
        x = rng.standard_normal(size=(n, 3, 224, 224)).astype(np.float32)
        desc = "VGG-19, fp32 NCHW, batch %d, 3x224x224, 1000 classes, momentum SGD" % n
    params = trainer.init_params(spec, seed=123)
    y = np.zeros((n, classes), np.float32)
    y[np.arange(n), rng.randint(0, classes, n)] = 1
    t = trainer.Trainer(spec, params, x.shape, classes, ctx, optimizer=opt)
    gx, gy = ndarray.array(x, ctx), ndarray.array(y, ctx)
    for _ in range(max(1, a.warmup)):
        t.step(gx, gy)
    t.sync()
    steps = a.steps
    if a.record:
        g = t.record_step(gx, gy)
        g.launch(t.stream)
        t.sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            g.launch(t.stream)
    else:
        t0 = time.perf_counter()
        for _ in range(steps):
            t.step(gx, gy)
    t.sync()
    dt = time.perf_counter() - t0
    print(json.dumps({"net": a.net, "workload": desc, "samples_per_s": n * steps / dt,
                      "ms_per_step": dt / steps * 1e3, "steps": steps, "warmup": a.warmup, "final_loss": t.loss_value(),
                      "recorded": bool(a.record),
                      "dtype": "f32 (matrix products and Winograd GEMMs as six bf16 x bf16 terms of exact operand splits, fp32 accumulation)"
                      if a.split_bf16 else "f32", "data": "synthetic"}))


if __name__ == "__main__":
    main()
