"""VGG-16 training throughput under device-memory budgets (one MI355X).

    python -m tsplit_amd.planbench [--budgets 0,8,7,6.5] [--fused] [--fused-pool] [--recompute] [--steps 5] [--warmup 2] [--batch 64]
    python -m tsplit_amd.planbench --max-batch [--budgets 8,16] [--fused] [--fused-pool] [--recompute]

For every budget (GiB; 0 = no limit) the planner chooses which activations leave for pinned
host memory (and, with --recompute, which BatchNorm / Relu outputs are dropped and computed again in
the backward sweep instead) and in how many micro-tensors the layers around them run; the budgeted executor
then trains batch-64 VGG-16 on synthetic data.  One JSON object per budget: samples/s, the
executor's measured peak, the plan.  With --max-batch the question is turned around, as in the
reference's batch-size sweeps (examples/imagenet_vgg.py:168-178): for every budget, the largest batch
that trains without a plan (everything resident) and the largest one the planner fits, and the
measured throughput and peak of the budgeted executor at the latter.
"""
import argparse
import json
import time

import numpy as np


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--budgets", default="0,8,7,6.5")
    ap.add_argument("--fused", action="store_true")
    ap.add_argument("--fused-pool", action="store_true", help="with --fused: the max pooling behind a BatchNorm+Relu pair joins it")
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--max-batch", action="store_true")
    ap.add_argument("--recompute", action="store_true", help="the plan may drop cheap tensors and compute them again")
    a = ap.parse_args()
    from . import ndarray, planner, trainer
    from .planned_trainer import PlannedTrainer, make_plan
    spec = trainer.vgg16_spec(1000, 224)
    params = trainer.init_params(spec, seed=123)
    if a.fused:
        spec = planner.fuse_spec(spec, pool=a.fused_pool, input_shape=(a.batch, 3, 224, 224))
    opt = ("momentum", 1e-4, 0.9)
    if a.max_batch:
        return max_batch_sweep(a, spec, params, opt)
    in_shape = (a.batch, 3, 224, 224)
    rng = np.random.RandomState(123)
    x = rng.standard_normal(size=in_shape).astype(np.float32)
    labels = np.zeros((a.batch, 1000), np.float32)
    labels[np.arange(a.batch), rng.randint(0, 1000, a.batch)] = 1.0
    ctx = ndarray.gpu(0)
    gx, gl = ndarray.array(x, ctx), ndarray.array(labels, ctx)
    for b in [float(v) for v in a.budgets.split(",")]:
        budget = None if b == 0 else int(b * (1 << 30))
        try:
            plan = make_plan(spec, in_shape, 1000, budget, opt, allow_recompute=a.recompute)
        except ValueError as e:
            print(json.dumps({"budget_GiB": b, "error": str(e)}), flush=True)
            continue
        t = PlannedTrainer(spec, params, in_shape, 1000, plan, ctx=ctx, optimizer=opt)
        for _ in range(a.warmup):
            t.step(gx, gl)
        t0 = time.perf_counter()
        for _ in range(a.steps):
            t.step(gx, gl)
        dt = (time.perf_counter() - t0) / a.steps
        d = plan.describe()
        print(json.dumps({"budget_GiB": b, "fused_bn_relu": a.fused, "fused_max_pool": bool(a.fused and a.fused_pool), "recompute": a.recompute, "samples_per_s": a.batch / dt, "ms_per_step": dt * 1e3,
                          "measured_peak_GiB": t.peak / planner.GiB, "planned_peak_GiB": d["peak_GiB"],
                          "estimated_ms_per_step": d["est_step_ms"],
                          "tensors_swapped": len(plan.swap), "swapped_GiB": sum(4 * int(np.prod(t.shapes[j])) for j in plan.swap) / planner.GiB,
                          "tensors_recomputed": len(plan.recompute),
                          "split": d["split"], "waits_for_memory": t.stall_events, "loss": t.loss_value()}), flush=True)
        del t


def max_batch_sweep(a, spec, params, opt):
    from . import ndarray, planner
    from .planned_trainer import PlannedTrainer, max_batch
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState(123)
    for b in [float(v) for v in a.budgets.split(",") if float(v) > 0]:
        budget = int(b * (1 << 30))
        resident, _ = max_batch(spec, (3, 224, 224), 1000, budget, opt, swap=False)
        planned, plan = max_batch(spec, (3, 224, 224), 1000, budget, opt, swap=True, allow_recompute=a.recompute)
        row = {"budget_GiB": b, "fused_bn_relu": a.fused, "fused_max_pool": bool(a.fused and a.fused_pool), "recompute": a.recompute, "max_batch_resident": resident,
               "max_batch_planned": planned}
        if plan is not None:
            in_shape = (planned, 3, 224, 224)
            x = rng.standard_normal(size=in_shape).astype(np.float32)
            labels = np.zeros((planned, 1000), np.float32)
            labels[np.arange(planned), rng.randint(0, 1000, planned)] = 1.0
            gx, gl = ndarray.array(x, ctx), ndarray.array(labels, ctx)
            t = PlannedTrainer(spec, params, in_shape, 1000, plan, ctx=ctx, optimizer=opt)
            t.step(gx, gl)
            t.sync()
            t0 = time.perf_counter()
            for _ in range(max(1, a.steps // 2)):
                t.step(gx, gl)
            t.sync()
            dt = (time.perf_counter() - t0) / max(1, a.steps // 2)
            row.update({"samples_per_s": planned / dt, "ms_per_step": dt * 1e3, "measured_peak_GiB": t.peak / planner.GiB,
                        "planned_peak_GiB": plan.describe()["peak_GiB"], "tensors_swapped": len(plan.swap),
                        "tensors_recomputed": len(plan.recompute),
                        "split": plan.describe()["split"], "loss": t.loss_value()})
            del t, gx, gl
        print(json.dumps(row), flush=True)


if __name__ == "__main__":
    main()
