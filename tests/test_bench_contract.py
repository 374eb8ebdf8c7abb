"""bench.py keeps the driver's contract: more than one GPU is refused with a message (the path has no collective), and a
run prints exactly one JSON line with the metric, the roofline of the dominant kernel and the CPU baseline."""
from __future__ import annotations

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    # a reduced matrix (the same kernel instance: K = 2048, 16-row units) so that the test takes seconds
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--rows", "65536", "--steps", "10", "--warmup", "2",
                        "--cpu-rows", "2048"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 10 and d["warmup"] == 2 and d["unit"] == "GB/s" and d["vs_baseline"] is None
    assert "workload" in d["config"] and "model" not in d["config"]
    rf = d["roofline"]
    assert rf["bound"] == "hbm" and rf["peak"] == 8000.0 and rf["unit"] == "GB/s"
    assert abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3 and 0.0 < rf["frac"] < 1.0
    assert abs(rf["achieved"] - rf["algorithmic_bytes"] / rf["avg_launch_us"] / 1e3) < 1.0
    cb = d["cpu_baseline"]
    assert cb["kind"] in ("port", "reference") and cb["cores"] >= 1 and cb["value"] > 0 and cb["unit"] == "GB/s" and cb["sample"]
    assert d["value"] > 100 * cb["value"] / 10                   # a GPU, not a fallback
    assert d["extra"]["max_err_over_sum_abs"] <= 1e-5           # the timed kernel's result was checked in the same run
