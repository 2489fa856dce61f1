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
    assert 0.3 < roof["frac"] < 1.0            # a measured fraction of the fp32 matrix peak, not a placeholder
    # the Winograd GEMM launches inside the timed steps add up to less than the steps themselves
    k = d["kernels"]["winograd_gemm"]
    assert 0 < k["ms_per_step"] < d["ms_per_step"]
