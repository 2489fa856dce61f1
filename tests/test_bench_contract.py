"""bench.py's command line and the JSON line it prints: one GPU only; on the GPU, a short run carries the
fields the measurement contract names (the whole-job figure, the step time it is derived from, and the roofline
object of the dominant kernel with its live-measured launch duration)."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, cwd=ROOT)
    assert r.returncode != 0
    assert "single-GPU" in (r.stdout + r.stderr)


@pytest.mark.gpu
def test_short_run_prints_the_contract_line():
    r = subprocess.run([sys.executable, BENCH, "--steps", "2", "--warmup", "1", "--no-cpu-baseline"], capture_output=True,
                       text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("{")][-1]
    d = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "kernels"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["warmup"] == 1 and d["higher_is_better"] is True
    assert d["unit"] == "samples/s" and d["dtype"] == "f32" and d["data"] == "synthetic" and d["vs_baseline"] is None
    assert "workload" in d["config"] and "VGG-16" in d["config"]["workload"] and d["config"]["global_batch"] == 64
    assert abs(d["value"] - 64 / (d["ms_per_step"] * 1e-3)) <= 1e-6 * d["value"]
    roof = d["roofline"]
    for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
        assert key in roof, key
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 157.3
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) <= 1e-9
    assert 0.25 < roof["frac"] < 1.0           # a measured fraction of the fp32 matrix peak, not a placeholder
    # the launches of the roofline's kernel inside the timed steps add up to less than the steps themselves
    assert roof["kernel"] == "winograd_fused" and roof["measured_in"] == "timed region"
    k = d["kernels"]["winograd_fused"]
    assert 0 < k["ms_per_step"] < d["ms_per_step"]


@pytest.mark.gpu
def test_run_with_the_cpu_leg_reports_the_same_loss_on_the_same_sample():
    """With the CPU leg, the line carries the CPU baseline (what was timed, on how many cores) and the first-step
    loss of the GPU path on the very sample the CPU path ran (16 of the seeded images, 4 micro-tensors on the first
    four convolutions): the two must agree within the 1e-3 relative bar of the end-to-end comparison."""
    r = subprocess.run([sys.executable, BENCH, "--steps", "2", "--warmup", "1"], capture_output=True, text=True, cwd=ROOT,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    d = json.loads([l for l in r.stdout.splitlines() if l.startswith("{")][-1])
    base = d["cpu_baseline"]
    for key in ("value", "unit", "cores", "kind", "sample"):
        assert key in base, key
    assert base["kind"] == "port" and base["unit"] == "samples/s" and base["cores"] >= 1 and base["value"] > 0
    assert d["gpu_vs_cpu_loss_rel_diff"] <= 1e-3, (d["gpu_loss_on_cpu_sample"], base["loss"])
    assert d["gpu_vs_cpu_loss_within_1e-3"] is True
    assert d["roofline"]["measured_in"] == "timed region"
    if "cpu_baseline_onednn" in d:          # the library path on the same sample: an independent third opinion
        assert abs(d["cpu_baseline_onednn"]["loss"] - base["loss"]) <= 1e-3 * abs(base["loss"])
