#!/usr/bin/env python3
"""Benchmark of the operator hot path: VGG-16 fp32 training steps on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

A step = forward + backward + momentum-SGD update of VGG-16 (13 conv3x3+BN+Relu, 5 max-pools,
3 bias-free FC; batch 64, 3x224x224, 1000 classes) issued through the C ABI on one stream,
with the four largest-resolution conv layers run as 4 batch micro-tensors.  Inputs,
labels and parameters are resident in HBM before the timed region starts.

Prints ONE JSON line.  Besides the contract fields it carries
  roofline      the single kernel with the largest share of the step (the 36-GEMM kernel inside the
                Winograd routine): executed FLOP per launch / mean launch time, measured with HIP event
                pairs the library records on the compute stream around every one of its launches inside
                the timed region (the only events there).
                Layers that run through the Winograd routine are several kernels per call (two
                transforms around 36 GEMMs); they are listed under `kernels` with the rate of the
                direct algorithm's FLOP count (which may exceed the MFMA peak: a quarter of those
                multiplications are executed) and are not candidates here
  kernels       the same figures for every operator class (TFLOP/s or GB/s), from one event per operator
                call over a second pass of K steps right after the timed region (those events cost
                about 3 us each, 0.9 ms a step: instrumented_ms_per_step shows the step with them)
  cpu_baseline  the numpy CPU oracle timed on this host on a bounded sample of the workload
  cpu_baseline_onednn  the same sample through PyTorch-CPU's bundled oneDNN (a library figure
                beside the oracle's; the reference's own dnnl build cannot be compiled here)
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS_FP32_MFMA = 157.3
PEAK_TFLOPS_BF16_MFMA = 2500.0   # dense bf16 matrix peak
PEAK_HBM_GBS = 8000.0
# Kernel names (as rocprofv3 prints them) behind the operator classes that can be the step's largest
# single kernel; their HBM bytes per launch are read from the counter summary under profiles/.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "vgg16_b64_train_step_hbm_traffic.txt")
TRAFFIC_PROFILE_FUSED = os.path.join(ROOT, "profiles", "vgg16_b64_fused_bn_relu_train_step_hbm_traffic.txt")      # bench.py --fused
TRAFFIC_PROFILE_SPLIT = os.path.join(ROOT, "profiles", "vgg16_b64_split_bf16_train_step_hbm_traffic.txt")          # --split-bf16
TRAFFIC_PROFILE_FUSED_SPLIT = os.path.join(ROOT, "profiles", "vgg16_b64_fused_split_bf16_train_step_hbm_traffic.txt")
TRAFFIC_KERNELS = {
    "conv_fwd_128x128": ("conv_tap_kernel<128, 128, 2, 2, false",),
    "conv_bwd_data_128x128": ("conv_tap_kernel<128, 128, 2, 2, true",),
    "conv_fwd_64x256": ("conv_tap_kernel<64, 256, 1, 4, false",),
    "conv_bwd_data_64x256": ("conv_tap_kernel<64, 256, 1, 4, true",),
    "conv_bwd_filter_128x128": ("conv_wgrad_tap_kernel<128, 128",),
    "winograd_gemm": ("wino_gemm_kernel<128, 128>",),
    "winograd_filter_grad_gemm": ("wino_grad_gemm_kernel<3>",),
    "winograd_gemm_64_rows": ("wino_gemm_kernel<64, 256>",),
    "winograd_fused": ("wino_fused_kernel<",),
    "winograd_filter_grad_fused": ("wino_fgrad_fused_kernel",),
    "winograd_gemm_split_bf16": ("wino_gemm_split_kernel",),
    "winograd_filter_grad_gemm_split_bf16": ("wino_grad_gemm_split_kernel<3>",),
}


def traffic_bytes_per_launch(tag, profile=TRAFFIC_PROFILE):
    """HBM bytes one launch of the class's kernel moves (read + write, mean over the launches of a step),
    from the FETCH_SIZE / WRITE_SIZE summary committed under profiles/ (columns: kernel, launches, read MB,
    write MB; several variants of one kernel are averaged by launch count).  None when the summary does
    not list the kernel: the figure is never a constant typed in here."""
    names = TRAFFIC_KERNELS.get(tag)
    if not names or not os.path.exists(profile):
        return None
    launches = total = 0.0
    with open(profile) as f:
        for line in f:
            if not any(line.startswith(n) for n in names):
                continue
            cols = line.split()
            try:
                n, rd, wr = float(cols[-3]), float(cols[-2]), float(cols[-1])
            except (ValueError, IndexError):
                continue
            launches += n
            total += n * (rd + wr) * 1e6
    return total / launches if launches else None


MFMA_PROFILE = os.path.join(ROOT, "profiles", "vgg16_b64_train_step_mfma_counters.txt")
MFMA_PROFILE_FUSED = os.path.join(ROOT, "profiles", "vgg16_b64_fused_bn_relu_train_step_mfma_counters.txt")       # bench.py --fused


def mfma_counters_per_launch(tag, profile=MFMA_PROFILE):
    """(FLOP the matrix pipes executed per launch, MFMA-busy %) of the class's kernel, from the rocprofv3 counter
    summary committed under profiles/ (SQ_INSTS_VALU_MFMA_MOPS_F32 x 512 and the MfmaUtil expression; columns:
    kernel, launches, avg us, MFMA GFLOP, TFLOP/s, of 157.3, MFMA busy %), averaged by launch count over the
    kernel's variants.  (None, None) when the summary does not list the kernel."""
    names = TRAFFIC_KERNELS.get(tag)
    if not names or not os.path.exists(profile):
        return None, None
    launches = flop = busy = 0.0
    with open(profile) as f:
        for line in f:
            if not any(line.startswith(n) for n in names):
                continue
            cols = line.split()
            try:
                n, g, b = float(cols[-6]), float(cols[-4]), float(cols[-1])
            except (ValueError, IndexError):
                continue
            launches += n
            flop += n * g * 1e9
            busy += n * b
    return (flop / launches, busy / launches) if launches else (None, None)


def vgg_workload(batch, seed=123):
    from tsplit_amd import trainer
    rng = np.random.RandomState(seed)
    spec = trainer.vgg16_spec(1000, 224)
    params = trainer.init_params(spec, seed=seed, scheme="he")
    x = rng.standard_normal(size=(batch, 3, 224, 224)).astype(np.float32)
    labels = np.zeros((batch, 1000), np.float32)
    labels[np.arange(batch), rng.randint(0, 1000, batch)] = 1.0
    conv_idx = [i for i, l in enumerate(spec) if l[0] == "conv"]
    split = {i: 4 for i in conv_idx[:4]}          # the two 224x224 and the two 112x112 layers
    return spec, params, x, labels, split


def cpu_baseline(sample_batch=16, seed=123):
    """The numpy oracle (float64, as the reference's numpy path computes) on `sample_batch`
    images of the same seeded workload: one forward+backward+momentum step."""
    from oracle import nets, ops
    spec, params, x, labels, _ = vgg_workload(sample_batch, seed)
    vel = {k: np.zeros_like(v) for k, v in params.items()}
    t0 = time.perf_counter()
    loss, _, grads = nets.forward_backward(spec, params, x, labels, eps=0.01)
    for k in params:
        ops.momentum_update(params[k], grads[k], vel[k], 0.01, 0.9)
    dt = time.perf_counter() - t0
    try:
        import threadpoolctl
        cores = max([p.get("num_threads", 1) for p in threadpoolctl.threadpool_info()] or [1])
    except Exception:
        cores = os.cpu_count() or 1
    return {"value": sample_batch / dt, "unit": "samples/s", "cores": int(cores), "kind": "port", "loss": loss,
            "sample": "one VGG-16 fwd+bwd+momentum step on %d of the 64 seeded images, numpy oracle in float64 "
                      "(%.1f s, loss %.4f)" % (sample_batch, dt, loss)}


def gpu_loss_on_sample(ctx, sample_batch=16, seed=123):
    """First-step loss of the GPU path on the sample the CPU baselines run (untimed)."""
    from tsplit_amd import ndarray, trainer
    spec, params, x, labels, split = vgg_workload(sample_batch, seed)
    t = trainer.Trainer(spec, params, x.shape, 1000, ctx, optimizer=("momentum", 0.01, 0.9), split=split)
    t.forward(ndarray.array(x, ctx), ndarray.array(labels, ctx))
    return t.loss_value()


def cpu_baseline_onednn(sample_batch=16, seed=123):
    """The same step on the same seeded sample through oneDNN as bundled with PyTorch-CPU
    (conv / batch-norm / pooling / matmul primitives, fp32, all host cores): the closest
    available stand-in for the reference's dnnl CPU operator build (src/dnnl_ops), whose
    oneDNN 1.x sources cannot be compiled against the library versions on this machine.
    Returns None when torch is not importable."""
    try:
        import torch
        import torch.nn.functional as F
    except Exception:
        return None
    spec, params, x, labels, _ = vgg_workload(sample_batch, seed)
    torch.set_num_threads(os.cpu_count() or 1)
    P = {k: torch.tensor(v, requires_grad=True) for k, v in params.items()}
    vel = {k: torch.zeros_like(v) for k, v in P.items()}
    xt, yt = torch.tensor(x), torch.tensor(labels)

    def step(update=True):
        h = xt
        for layer in spec:
            kind = layer[0]
            if kind == "conv":
                h = F.conv2d(h, P[layer[1] + "_weight"], padding=layer[5], stride=layer[6])
            elif kind == "bn":
                h = F.batch_norm(h, None, None, P[layer[1] + "_scale"].reshape(-1), P[layer[1] + "_bias"].reshape(-1),
                                 training=True, eps=0.01)
            elif kind == "relu":
                h = F.relu(h)
            elif kind == "maxpool":
                h = F.max_pool2d(h, layer[1], layer[3], layer[2])
            elif kind == "flatten":
                h = h.reshape(h.shape[0], -1)
            elif kind == "fc":
                h = h @ P[layer[1] + "_weight"]
        loss = -(yt * F.log_softmax(h, dim=1)).sum(dim=1).mean()
        loss.backward()
        with torch.no_grad():
            for k, p in P.items():
                if update:
                    vel[k].mul_(0.9).sub_(p.grad, alpha=0.01)
                    p.add_(vel[k])
                p.grad = None
        return float(loss.detach())
    step(update=False)           # warm-up: primitive creation, allocator; parameters stay as seeded
    t0 = time.perf_counter()
    loss = step()
    dt = time.perf_counter() - t0
    return {"value": sample_batch / dt, "unit": "samples/s", "cores": int(torch.get_num_threads()), "kind": "library",
            "loss": loss, "sample": "one VGG-16 fwd+bwd+momentum step on %d of the 64 seeded images, PyTorch-CPU %s with its "
                      "bundled oneDNN, fp32 (%.2f s, loss %.4f)" % (sample_batch, torch.__version__, dt, loss)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-split", action="store_true")
    ap.add_argument("--no-events", action="store_true", help="time the steps without per-launch events")
    ap.add_argument("--fused", action="store_true",
                    help="run every BatchNorm+Relu pair (and the max pooling behind it, where one follows) through the fused "
                         "symbols, let every convolution hand its output's statistics to the BatchNorm behind it and "
                         "update all parameters in one launch (symbols outside the reference's ABI)")
    ap.add_argument("--split-bf16", action="store_true",
                    help="opt-in, outside the reference's ABI and outside the default path's fp32 matrix instructions: the "
                         "Winograd GEMMs of layers with more than 64 channels on both sides take each fp32 product as six "
                         "bf16 x bf16 products of the operands' exact three-term splits, accumulated in fp32")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build is single-GPU by design (no collectives, no sharding); run with --gpus 1. "
                 "The one-GPU figure is the whole-job throughput.")

    from tsplit_amd import gpu_links as L, ndarray, trainer
    from tsplit_amd.timing import EventTimer
    ctx = ndarray.gpu(0)
    spec, params, x, labels, split = vgg_workload(a.batch)
    if a.no_split:
        split = {}
    timer = None if a.no_events else EventTimer(ctx, chained=True)
    L.split_bf16(a.split_bf16)
    t = trainer.Trainer(spec, params, x.shape, 1000, ctx, optimizer=("momentum", 1e-4, 0.9), split=split, timer=timer,
                        fuse_bn_relu=a.fused, conv_bn_stats=a.fused, multi_tensor_update=a.fused, fuse_max_pool=a.fused)
    gx, gy = ndarray.array(x, ctx), ndarray.array(labels, ctx)      # resident before timing
    for _ in range(a.warmup):
        t.step(gx, gy)
    t.sync()
    # The timed region: K steps with event pairs only around the launches of the step's largest kernel, the
    # one-kernel Winograd convolution of the layers with up to 256 channels (forward and data gradient; recorded
    # by the library on the compute stream; 30 launches per step, about 5 us per pair).  The events of the routine's other GEMM kernels
    # and the per-call events behind the kernels{} table (about 3 us per launch, 0.9 ms over the ~400 launches of
    # a step) bracket a second pass of K steps after the timed region.
    dominant_kind = 3 if a.split_bf16 else 5
    if timer:
        L.winograd_gemm_timing(True, kind=dominant_kind)
    t0 = time.perf_counter()
    for _ in range(a.steps):
        t.step(gx, gy)
    t.sync()
    dt = time.perf_counter() - t0
    gemm_times = {dominant_kind: L.winograd_gemm_times(kind=dominant_kind)} if timer else {}
    L.winograd_gemm_timing(False)
    if timer:
        timer.enabled = True
        L.winograd_gemm_timing(True)
        t1 = time.perf_counter()
        for _ in range(a.steps):
            t.step(gx, gy)
        t.sync()
        dt_instrumented = time.perf_counter() - t1
        for kind in range(7):
            if kind != dominant_kind:
                gemm_times[kind] = L.winograd_gemm_times(kind=kind)
        L.winograd_gemm_timing(False)
    loss = float(t.loss.asnumpy()[0])
    ms_per_step = dt / a.steps * 1e3

    out = {
        "metric": "train samples/s, fp32, 1 MI355X; conv MFMA util %; BN/relu HBM GB/s",
        "value": a.batch * a.steps / dt, "unit": "samples/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32 (Winograd GEMM products of wide layers as six bf16 x bf16 terms of exact operand splits, fp32 accumulation)"
                 if a.split_bf16 else "f32", "data": "synthetic",
        "config": {"workload": "VGG-16 training step (fwd+bwd+momentum SGD), fp32 NCHW, batch %d, 3x224x224, "
                               "1000 classes, He init, %s%s" % (a.batch, "4 batch micro-tensors on the 4 largest conv layers"
                                                                if split else "no micro-tensor split",
                                                                (", BatchNorm+Relu pairs fused (with the max pooling behind them where one follows), BatchNorm statistics from the convolutions' epilogues, one optimizer launch" if a.fused else "")
                                                                + (", split-bf16 products in the wide layers' Winograd GEMMs" if a.split_bf16 else "")),
                   "global_batch": a.batch, "final_loss": loss},
    }
    if timer:
        k = timer.collect()
        kernels = {}
        for tag, d in sorted(k.items(), key=lambda kv: -kv[1]["ms_total"]):
            peak = PEAK_TFLOPS_FP32_MFMA if d["unit"] == "flop" else PEAK_HBM_GBS
            kernels[tag] = {"calls_per_step": d["calls"] / a.steps, "ms_per_step": d["ms_total"] / a.steps,
                            "ms_avg": d["ms_avg"], "achieved": d["rate"],
                            "unit": "TFLOP/s" if d["unit"] == "flop" else "GB/s", "frac": d["rate"] / peak}
            if tag.endswith("_winograd"):
                # several kernels per call, and a quarter of the direct algorithm's multiplications are
                # executed: the rate below is on the direct FLOP count and is no fraction of any peak
                del kernels[tag]["frac"]
                kernels[tag]["note"] = ("several kernels per call; rate of the direct algorithm's FLOP count, of which the "
                                        "Winograd GEMMs execute a quarter (see winograd_gemm / winograd_filter_grad_gemm)")
            if "bytes" in d:      # near the ridge: both fractions
                kernels[tag]["hbm_achieved_gbs"] = d["bytes"] / (d["ms_total"] * 1e-3) / 1e9
                kernels[tag]["hbm_frac"] = kernels[tag]["hbm_achieved_gbs"] / PEAK_HBM_GBS
        # the GEMM kernels inside the Winograd calls, timed by the library with event pairs on the
        # compute stream around each launch; their work is the FLOP they execute
        wino_exec_flop = 0.0
        for tag, kind in (("winograd_gemm", 0), ("winograd_filter_grad_gemm", 1), ("winograd_gemm_64_rows", 2), ("winograd_fused", 5),
                          ("winograd_filter_grad_fused", 6)):
            launches, ms, flop, nbytes = gemm_times[kind]
            if launches:
                wino_exec_flop += flop
                k[tag] = {"calls": launches, "ms_total": ms, "ms_avg": ms / launches, "work": flop,
                          "work_per_call": flop / launches, "rate": flop / (ms * 1e-3) / 1e12, "unit": "flop"}
                kernels[tag] = {"calls_per_step": launches / a.steps, "ms_per_step": ms / a.steps, "ms_avg": ms / launches,
                                "achieved": k[tag]["rate"], "unit": "TFLOP/s", "frac": k[tag]["rate"] / PEAK_TFLOPS_FP32_MFMA,
                                "note": "one kernel inside the *_winograd calls above (its time is part of theirs); "
                                        "executed FLOP"}
                if kind == 5:
                    # forward / data gradient of the layers with 64 channels on one side as ONE kernel (transforms inside,
                    # the transformed tensors never leave the chip): its time is the whole call's, its bytes the activations'
                    kernels[tag]["hbm_achieved_gbs"] = nbytes / (ms * 1e-3) / 1e9
                    kernels[tag]["hbm_frac"] = kernels[tag]["hbm_achieved_gbs"] / PEAK_HBM_GBS
                    kernels[tag]["note"] = ("the whole forward / data-gradient call of the layers with 64 channels on one side: one kernel "
                                            "with the Winograd transforms inside; executed FLOP (2 * 36 * O * C * tiles), and the "
                                            "activations' and filter's bytes for hbm_*")
                if kind == 6:
                    # filter gradient of the layers with at most 128 channels as ONE kernel plus the final transform of
                    # the filter: both transforms on the way into LDS, products there
                    kernels[tag]["hbm_achieved_gbs"] = nbytes / (ms * 1e-3) / 1e9
                    kernels[tag]["hbm_frac"] = kernels[tag]["hbm_achieved_gbs"] / PEAK_HBM_GBS
                    kernels[tag]["note"] = ("the filter-gradient call of the layers with at most 128 channels but for its final 3x3 transform: "
                                            "one kernel with both Winograd transforms inside; executed FLOP (2 * 36 * O * C * tiles), and "
                                            "the activations', gradients' and partial sums' bytes for hbm_*")
                if kind == 2:
                    # 64 or 128 channels summed over on 64-row tiles: 16 - 21 executed FLOP per algorithmic byte, at
                    # the ratio of the two peaks (19.7), so both fractions are given
                    kernels[tag]["hbm_achieved_gbs"] = nbytes / (ms * 1e-3) / 1e9
                    kernels[tag]["hbm_frac"] = kernels[tag]["hbm_achieved_gbs"] / PEAK_HBM_GBS
                    kernels[tag]["note"] = ("the forward / data-gradient GEMMs of the layers that produce 64 channels (64 x 256 "
                                            "tiles) inside the *_winograd calls; executed FLOP, and algorithmic bytes for hbm_*")
        # the same GEMMs with split-bf16 products: six bf16 matrix instructions per fp32-equivalent product, so
        # the executed work is six times the GEMM's FLOP and the peak is the bf16 matrix peak
        for tag, kind in (("winograd_gemm_split_bf16", 3), ("winograd_filter_grad_gemm_split_bf16", 4)):
            launches, ms, flop, nbytes = gemm_times[kind]
            if launches:
                k[tag] = {"calls": launches, "ms_total": ms, "ms_avg": ms / launches, "work": 6 * flop,
                          "work_per_call": 6 * flop / launches, "rate": 6 * flop / (ms * 1e-3) / 1e12, "unit": "flop",
                          "peak": PEAK_TFLOPS_BF16_MFMA}
                kernels[tag] = {"calls_per_step": launches / a.steps, "ms_per_step": ms / a.steps, "ms_avg": ms / launches,
                                "achieved": k[tag]["rate"], "unit": "TFLOP/s", "frac": k[tag]["rate"] / PEAK_TFLOPS_BF16_MFMA,
                                "fp32_equivalent_tflops": flop / (ms * 1e-3) / 1e12,
                                "hbm_achieved_gbs": nbytes / (ms * 1e-3) / 1e9, "hbm_frac": nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                "note": "one kernel inside the *_winograd calls above; executed bf16 FLOP (six products per "
                                        "fp32-equivalent product) against the bf16 matrix peak, and algorithmic bytes for hbm_*"}
        kernels = dict(sorted(kernels.items(), key=lambda kv: -kv[1]["ms_per_step"]))
        dom = next(tag for tag in kernels if not tag.endswith("_winograd"))
        dd = k[dom]
        dom_peak = dd.get("peak", PEAK_TFLOPS_FP32_MFMA if dd["unit"] == "flop" else PEAK_HBM_GBS)
        out["roofline"] = {"kernel": dom, "bound": "mfma" if dd["unit"] == "flop" else "hbm",
                           "achieved": dd["rate"], "peak": dom_peak,
                           "unit": "TFLOP/s" if dd["unit"] == "flop" else "GB/s",
                           "frac": dd["rate"] / dom_peak,
                           "traffic": traffic_bytes_per_launch(dom, {(False, False): TRAFFIC_PROFILE, (True, False): TRAFFIC_PROFILE_FUSED,
                                                                     (False, True): TRAFFIC_PROFILE_SPLIT,
                                                                     (True, True): TRAFFIC_PROFILE_FUSED_SPLIT}[(a.fused, a.split_bf16)])
                           if split and a.batch == 64 else None,
                           "per_launch": dd["work_per_call"], "ms_avg": dd["ms_avg"],
                           # which pass the launch durations behind `achieved` come from: the timed region carries event
                           # pairs only for the kernel expected to be the largest; if another one turns out larger (other
                           # batch sizes, --fused, --no-split) its figures are those of the second, instrumented pass
                           "measured_in": "timed region" if dom == {5: "winograd_fused", 3: "winograd_gemm_split_bf16"}[dominant_kind]
                           else "second pass (one event per operator call)"}
        if split and a.batch == 64 and not a.split_bf16 and dd["unit"] == "flop":
            # what the matrix pipes executed per launch and the share of cycles they were busy, by counter
            # (committed summary of a rocprofv3 --pmc run of this command); per_launch above is arithmetic
            counted, busy = mfma_counters_per_launch(dom, MFMA_PROFILE_FUSED if a.fused else MFMA_PROFILE)
            out["roofline"]["per_launch_by_mfma_counter"] = counted
            out["roofline"]["mfma_busy_pct"] = busy
        # Conv utilisation, two ways.  The thin first layer (Cin*kH*kW = 27) is timed in bytes because
        # HBM bounds it, so its FLOP (forward and filter gradient) are added to both counts.
        conv = {tag: d for tag, d in k.items() if tag.startswith("conv_")}      # the Winograd GEMMs' time is inside these
        thin_flop = 0.0
        shape = x.shape
        for layer in spec:
            if layer[0] == "conv":
                if layer[2] * layer[4] * layer[4] <= 32:
                    thin_flop += a.steps * 2 * 2.0 * shape[0] * layer[3] * shape[2] * shape[3] * layer[2] * layer[4] ** 2
                shape = (shape[0], layer[3], shape[2], shape[3])
            elif layer[0] == "maxpool":
                shape = (shape[0], shape[1], shape[2] // 2, shape[3] // 2)
        conv_ms = sum(d["ms_total"] for d in conv.values())
        direct_flop = sum(d["work"] for tag, d in conv.items() if d["unit"] == "flop" and not tag.endswith("_winograd"))
        equivalent_flop = sum(d["work"] for d in conv.values() if d["unit"] == "flop") + thin_flop

        def pct(flop, ms):
            return 100.0 * flop / (ms * 1e-3) / 1e12 / PEAK_TFLOPS_FP32_MFMA if ms > 0 else None
        # executed: what the matrix pipe really multiplies (the Winograd calls count with their 36 GEMMs'
        # FLOP, the direct kernels with the algorithm's) over ALL conv time, transforms included
        # (with split-bf16 products part of the work runs on the bf16 matrix instruction: no single peak applies)
        out["conv_mfma_util_executed_pct"] = None if a.split_bf16 else pct(direct_flop + thin_flop + wino_exec_flop, conv_ms)
        # direct-equivalent: the direct algorithm's FLOP count of every layer over the same time; above 100
        # because the Winograd layers execute a quarter of it.  A throughput figure, not a utilisation
        out["conv_direct_equivalent_pct"] = pct(equivalent_flop, conv_ms)
        out["conv_effective_tflops"] = equivalent_flop / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else None
        # the direct kernels alone, whose executed FLOP are the algorithmic ones
        direct_ms = sum(d["ms_total"] for tag, d in conv.items() if d["unit"] == "flop" and not tag.endswith("_winograd"))
        if direct_ms > 0:
            out["conv_mfma_util_direct_kernels_pct"] = pct(direct_flop, direct_ms)
        out["kernels"] = kernels
        out["instrumented_ms_per_step"] = dt_instrumented / a.steps * 1e3
        out["timing_note"] = ("value and ms_per_step: K steps with event pairs around the launches of the roofline's kernel only (the "
                              "one-kernel Winograd convolution, wino_fused_kernel: its kernels{} entry and roofline come from "
                              "those); the other kernels{} entries, the routine's GEMM kernels included: a second "
                              "pass of K steps with one event per operator call, whose own cost shows in instrumented_ms_per_step")
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        # the same 16-image sample, same seeded parameters, once through the GPU path (forward of the first
        # step, 4 micro-tensors on the first four convolutions): the loss the CPU figures report beside it
        out["gpu_loss_on_cpu_sample"] = gpu_loss_on_sample(ctx)
        out["gpu_vs_cpu_loss_rel_diff"] = abs(out["gpu_loss_on_cpu_sample"] - out["cpu_baseline"]["loss"]) / abs(
            out["cpu_baseline"]["loss"])
        # the end-to-end bar of the benchmark configuration: the loss tracks the CPU path within 1e-3 relative
        out["gpu_vs_cpu_loss_within_1e-3"] = bool(out["gpu_vs_cpu_loss_rel_diff"] <= 1e-3)
        onednn = cpu_baseline_onednn()
        if onednn:
            out["cpu_baseline_onednn"] = onednn
    print(json.dumps(out))


if __name__ == "__main__":
    main()
