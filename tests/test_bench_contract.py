"""bench.py's contract with its driver: one GPU only, and one JSON line that carries the metric, the roofline of the
dominant kernel and the CPU baseline, for the three types the metric names."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0
    assert "one GPU" in done.stderr and not done.stdout.strip()


@pytest.mark.gpu
def test_one_line_with_roofline_and_cpu_baseline():
    """A short run (3 steps, the other workloads left out): the line parses, names the headline workload, and every
    figure in it follows from the others (achieved = ops / kernel time, frac = achieved / peak)."""
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "3", "--warmup", "1",
                           "--no-others", "--no-vendor", "--no-ceiling", "--spin-up-ms", "20"],
                          capture_output=True, text=True, timeout=600)
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "spin_up_ms"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 1 and line["unit"] == "gso/s"
    assert line["dtype"] == "i8" and line["vs_baseline"] is None and "M=8192 N=8192 K=8192" in line["config"]["workload"]
    roofline = line["roofline"]
    assert roofline["bound"] == "mfma" and roofline["peak"] == 5000.0 and roofline["unit"] == "TFLOP/s"
    ops = 2.0 * 8192 ** 3
    assert abs(roofline["achieved"] - ops / (line["kernel_ms"] * 1e-3) / 1e12) < 1e-6 * roofline["achieved"]
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-9 and 0.2 < roofline["frac"] < 1.0
    assert abs(line["value"] - ops / (line["ms_per_step"] * 1e-3) / 1e9) < 1e-6 * line["value"]
    assert line["kernel_ms"] <= line["ms_per_step"] * 1.05
    assert set(roofline["by_dtype"]) == {"i8", "bf16", "e4m3"} and "frac_f16" in roofline["by_dtype"]["e4m3"]
    baseline = line["cpu_baseline"]
    assert baseline["kind"] == "reference" and baseline["cores"] >= 1 and baseline["value"] > 0 and baseline["unit"] == "gso/s"
    assert set(baseline["by_dtype"]) == {"i8", "bf16", "e4m3"}
