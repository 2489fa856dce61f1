"""The branched example networks trained under device-memory budgets (one MI355X): the budgeted tape
executor of tape_budget.py on ResNet-50 (batch 64), Inception-v4 (batch 32) and the Transformer (batch 32).

    python -m tsplit_amd.tapebench --net resnet50|inception_v4|transformer [--fractions 0,0.75,0.5,0.35] [--steps 4] [--warmup 1] [--no-recompute] [--tune | --lead L --hold H]
    python -m tsplit_amd.tapebench --net resnet50|inception_v4 --max-batch [--budgets 8,16] [--no-recompute] [--tune]
    python -m tsplit_amd.tapebench --net transformer --fractions 0.5,0.35,0.25,0.15 --split 4 [--split-always]

For every fraction f (0 = no limit) the budget is the leaves (parameters, their gradients' room is part
of the replay, inputs, constants) plus f times what the operators' values and gradients take at the
unplanned peak; the planner picks what is dropped and computed again and what leaves for pinned host memory
(only the latter with --no-recompute), the executor trains on synthetic data.  One JSON object per budget: samples/s, the pool's measured peak over its level before the run,
the replayed peak, values sent away, host waits per step.  --lead and --hold set the schedule (how many operators ahead of
its reader a value starts coming back, for how many operators a leaving value keeps its memory while its copy runs);
with --tune the run first trains two steps under each of a few schedules and keeps the fastest.  With --max-batch the question is turned
around, as in the reference's batch-size sweeps per policy (examples/imagenet_resnet.py:139-154): for
every budget in GiB, the largest batch that trains with everything resident and the largest one the
planner fits, and the measured throughput at the latter.
"""
import argparse
import json
import time

import numpy as np


def _net(name, batch=None):
    """-> (builder(batch), numpy inputs(batch, rng), default batch, description)"""
    from . import workloads
    if name == "resnet50":
        def build_for(n):
            return lambda t, b, c: workloads.resnet(t, b, c["x"], c["y"])

        def inputs_for(n, rng):
            y = np.zeros((n, 1000), np.float32)
            y[np.arange(n), rng.randint(0, 1000, n)] = 1
            return {"x": rng.standard_normal((n, 3, 224, 224)).astype(np.float32), "y": y}
        return build_for, inputs_for, 64, "ResNet-50, fp32 NCHW, 3x224x224, 1000 classes"
    if name == "inception_v4":
        def build_for(n):
            return lambda t, b, c: workloads.inception_v4(t, b, c["x"], c["y"])

        def inputs_for(n, rng):
            y = np.zeros((n, 1000), np.float32)
            y[np.arange(n), rng.randint(0, 1000, n)] = 1
            return {"x": rng.standard_normal((n, 3, 299, 299)).astype(np.float32), "y": y}
        return build_for, inputs_for, 32, "Inception-v4, fp32 NCHW, 3x299x299, 1000 classes"
    if name == "transformer":
        def cfg_for(n):
            return workloads.TransformerConfig(batch=n, mask_value=0.0, embed_std=0.0002, pos_amplitude=0.003)

        def build_for(n):
            cfg = cfg_for(n)
            return lambda t, b, c: workloads.transformer(t, b, cfg, c["xs"], c["yi"], c["yo"])

        def inputs_for(n, rng):
            cfg = cfg_for(n)
            return {"xs": rng.randint(1, cfg.vocab, size=(n, cfg.len1)).astype(np.float32),
                    "yi": rng.randint(1, cfg.vocab, size=(n, cfg.len2)).astype(np.float32),
                    "yo": rng.randint(1, cfg.vocab, size=(n, cfg.len2)).astype(np.float32)}
        return build_for, inputs_for, 32, "Transformer 6+6 blocks, d_model 512, 8 heads, FFN 2048, length 256, vocab 32000"
    raise ValueError(name)


def _measure(build, inputs, budget, steps, warmup, lr, recompute=True, lead=3, hold=1, tune=False, fused=False,
             piece_build=None, pieces=1, split_always=False):
    from . import tape_budget as tb, workloads
    from .gpu_memory_manager import pool_state
    base = pool_state().used
    run = tb.BudgetedRun(build, inputs, workloads.ParamStore(123), budget, lead=lead, track_pool=True, recompute=recompute,
                         hold=hold, fuse_bn_relu=fused, piece_build=piece_build, pieces=pieces, split_always=split_always)
    tuned = None
    if tune and budget is not None:
        best, timings, _ = run.tune(lr)
        tuned = {"lead": best[0], "hold": best[1], "ms_per_schedule": {"%d,%d" % k: round(v, 2) for k, v in timings.items()}}
        run.state.peak_used = 0          # the pool's peak below is that of the schedule kept
    for _ in range(warmup):
        run.step(lr)
    run.sync()
    waits0 = run.state.host_waits
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = run.step(lr)
    run.sync()
    dt = (time.perf_counter() - t0) / steps
    n = next(iter(inputs.values())).shape[0]
    d = run.plan.describe()
    gib = float(1 << 30)
    return {"samples_per_s": n / dt, "ms_per_step": dt * 1e3, "measured_peak_GiB": (run.state.peak_used - base) / gib,
            "planned_peak_GiB": d["peak_GiB"], "unplanned_peak_GiB": d["unplanned_peak_GiB"], "values_away": d["away"],
            "away_GiB": sum(run.ops[i].bytes for i in run.plan.away) / gib, "values_recomputed": len(run.plan.redo),
            "recomputed_GiB": sum(run.ops[i].bytes for i in run.plan.redo) / gib,
            "host_waits_per_step": (run.state.host_waits - waits0) / steps, "loss": float(loss.value.asnumpy()[0]),
            "lead": run.plan.lead, "hold": run.plan.hold, "tuned": tuned,
            # operators from split_from on (of operators_whole in the graph) run per batch micro-tensor, `pieces` of them
            "split_from": run.plan.split_from, "pieces": run.plan.pieces,
            "operators_whole": len(run.piece_calls) if run.piece_calls else len(run.ops)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--net", default="resnet50", choices=["resnet50", "inception_v4", "transformer"])
    ap.add_argument("--fractions", default="0,0.75,0.5,0.35")
    ap.add_argument("--budgets", default="8,16")
    ap.add_argument("--batch", type=int, default=0)
    ap.add_argument("--steps", type=int, default=4)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--lr", type=float, default=1e-4)
    ap.add_argument("--max-batch", action="store_true")
    ap.add_argument("--no-recompute", action="store_true", help="the plan may only send values to the host")
    ap.add_argument("--lead", type=int, default=3, help="operators ahead of its first reader at which a value starts coming back")
    ap.add_argument("--fused", action="store_true",
                    help="BatchNorm + Relu pairs as one node each (TSplit_BatchNormRelu): the BatchNorm output is never written")
    ap.add_argument("--tune", action="store_true",
                    help="train two steps under each of a few (lead, hold) schedules first and keep the fastest")
    ap.add_argument("--hold", type=int, default=1, help="operators behind its last reader after which a leaving value is released")
    ap.add_argument("--split", type=int, default=0,
                    help="the planner may run the end of the graph on this many batch micro-tensors when whole values cannot meet the budget")
    ap.add_argument("--split-always", action="store_true", help="with --split: run a stretch per micro-tensor under every budget")
    a = ap.parse_args()
    from . import tape_budget as tb
    build_for, inputs_for, default_batch, desc = _net(a.net)
    rng = np.random.RandomState(123)
    if a.max_batch:
        for b in [float(v) for v in a.budgets.split(",")]:
            budget = int(b * (1 << 30))

            one = {k: v.shape[1:] for k, v in inputs_for(1, np.random.RandomState(0)).items()}

            def shapes_for(n):
                return {k: (n,) + tail for k, tail in one.items()}
            resident, _ = tb.max_batch(build_for, shapes_for, budget, planned=False, fuse_bn_relu=a.fused)
            planned, p = tb.max_batch(build_for, shapes_for, budget, planned=True, recompute=not a.no_recompute,
                                      fuse_bn_relu=a.fused)
            row = {"net": a.net, "workload": desc, "budget_GiB": b, "recompute": not a.no_recompute,
                   "max_batch_resident": resident, "max_batch_planned": planned}
            if p is not None:
                row.update(_measure(build_for(planned), inputs_for(planned, rng), budget, max(1, a.steps // 2), 1, a.lr,
                                    not a.no_recompute, a.lead, a.hold, a.tune, a.fused))
            print(json.dumps(row), flush=True)
        return
    n = a.batch or default_batch
    inputs = inputs_for(n, rng)
    build = build_for(n)
    ops, leaves = tb.record(build, {k: v.shape for k, v in inputs.items()}, a.fused)
    free_peak = tb.replay(ops, leaves)[0]
    for f in [float(v) for v in a.fractions.split(",")]:
        budget = None if f == 0 else leaves + int((free_peak - leaves) * f)
        row = {"net": a.net, "workload": desc + ", batch %d" % n, "fraction": f,
               "budget_GiB": None if budget is None else budget / float(1 << 30), "recompute": not a.no_recompute,
               "fused_bn_relu": a.fused}
        try:
            row.update(_measure(build, inputs, budget, a.steps, a.warmup, a.lr, not a.no_recompute, a.lead, a.hold, a.tune, a.fused,
                                build_for(n // a.split) if a.split > 1 else None, max(1, a.split), a.split_always))
        except ValueError as e:
            row["error"] = str(e)
        print(json.dumps(row), flush=True)


if __name__ == "__main__":
    main()
