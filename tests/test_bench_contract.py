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
                        "--cpu-rows", "2048", "--cpu-seconds", "3", "--weight-sets", "8"], capture_output=True, text=True, timeout=900)
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
    assert rf["traffic"] is None and rf["traffic_source"] is None   # counters exist for the full-size workload only
    assert "timed" in d["config"]["workload"] and "generator" in d["config"]
    # the timed region: blocks of `steps` launches until 50 ms have been timed, the median block reported
    lo, hi = d["extra"]["block_us_per_step_min_max"]
    assert lo <= d["ms_per_step"] * 1e3 <= hi
    # a read-only kernel of the library's own as the yardstick, in its four access patterns
    assert len(d["extra"]["read_probe_GBps"]) == 8 and d["extra"]["plain_stream_read_GBps"] == max(d["extra"]["read_probe_GBps"].values())
    # the CPU reference configuration, one thread and all
    c1 = cb["config1_2048x2048"]
    assert c1["threads_1"]["us"] > 0 and c1["compressed_bytes"] > 0 and f"threads_{cb['cores']}" in c1
    # the other configurations of the path, measured in the same run
    cf = d["extra"]["configs"]
    for key in ("lm_head_batch4", "gemv_512x2048", "gemv_2048x512", "moe_layer_batch1_graph", "moe_prefill_T2048", "moe_prefill_T8192",
                "decode_step"):
        assert key in cf, key
    assert cf["decode_step"]["weight_sets"] == 8
    for b in ("batch1", "batch4", "batch16"):
        e = cf["decode_step"][b]
        assert e["us"] > 0 and e["bf16_us"] > 0 and e["eager_equals_graph"] and 0 < e["frac_of_hbm_peak"] < 1
        # both stock-kernel comparators up to four tokens, the speed-up against the faster of them
        best = min(e["bf16_us"], e["bf16_static_ids_us"]) if b != "batch16" else e["bf16_us"]
        assert abs(e["speedup_vs_bf16"] - best / e["us"]) < 0.02
    # the kernel name comes from the library's dispatch, the stock GEMV is timed like the headline kernel
    assert rf["kernel"].startswith("k_w64_mmv<bf16_t, 4, 1, ") and "blas_timing" in d["extra"]
    b4 = cf["lm_head_batch4"]
    assert b4["units_of_16_rows"]["kernel"].startswith("k_w64_mmv<bf16_t, 4, 4, ") and b4["matrix_core_tiles"]["us"] > 0
    e4 = cf["decode_step"]["experts_4bit_code"]
    assert e4["batch1"]["us"] > 0 and e4["batch4"]["us"] > 0 and 1.0 < e4["expert_bytes_vs_tiles"] < 1.2
    for T in (2048, 8192):
        e = cf[f"moe_prefill_T{T}"]
        assert 0 < e["frac_of_bf16_mfma_peak"] < 1 and e["weight_decode_GBps"] > 0


def test_counter_traffic_comes_from_the_committed_profile():
    sys.path.insert(0, ROOT)
    import bench

    t = bench.measured_traffic(248320, 2048)
    assert t is not None and 0.98 * 686_670_516 < t < 1.10 * 686_670_516
    assert bench.measured_traffic(65536, 2048) is None
    assert os.path.exists(os.path.join(ROOT, bench.TRAFFIC_PROFILE))
