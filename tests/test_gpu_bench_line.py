"""bench.py on the GPU: a short run prints exactly one JSON line with the fields the measurement contract
names, and its figures are consistent with each other."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, lines
    return json.loads(lines[0])


def test_headline_line_short_run():
    b = _run("--steps", "60", "--warmup", "10", "--samples", "8960", "--cpu-baseline-seconds", "2",
             "--other-configs", "dense")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in b, key
    assert b["n_gpus"] == 1 and b["steps"] == 60 and b["warmup"] == 10 and b["higher_is_better"] is True
    assert b["unit"] == "samples/s" and b["dtype"] == "f32" and b["vs_baseline"] is None
    assert "workload" in b["config"] and "model" not in b["config"]
    # value = samples / time; 60 full batches of 128 in the timed region
    assert b["value"] == pytest.approx(60 * 128 / (b["ms_per_step"] * 60 / 1e3), rel=1e-6)
    r = b["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert r["frac"] == pytest.approx(r["achieved"] / r["peak"], rel=1e-9) and 0.0 < r["frac"] < 1.0
    assert r["achieved"] == pytest.approx(r["algorithmic_bytes_per_launch"] / (r["avg_launch_us"] * 1e-6) / 1e9, rel=1e-6)
    # the dominant kernel's duration comes from events its launches carry (dispatch begin to end): nothing subtracted
    k = b["kernels"]["train_fused"]
    assert k["events"] == "carried" and k["avg_us"] == k["raw_avg_us"] == r["avg_launch_us"]
    assert b["kernels"]["forward"]["events"] == "bracket" and b["kernels"]["forward"]["avg_us"] < b["kernels"]["forward"]["raw_avg_us"]
    # the counter summary in profiles/ belongs to the kernel sources of this tree
    assert r["traffic"] is not None, r["traffic_note"]
    assert 0.5 * r["algorithmic_bytes_per_launch"] < r["traffic"] < 2 * r["algorithmic_bytes_per_launch"]
    w = b["windows"]
    assert w["count"] >= 3 and w["ms_per_step_min"] <= w["ms_per_step_median"] <= w["ms_per_step_max"]
    assert b["ms_per_step"] == pytest.approx(w["ms_per_step_median"], rel=1e-9)
    c = b["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["unit"] == "samples/s"
    assert b["value"] > c["value"]
    assert set(c["ms_per_step_by_function"]) == {"forward_blas", "softmax_numpy", "traces_and_weights", "bias", "mask"}
    assert sum(c["ms_per_step_by_function"].values()) <= c["ms_per_step"] * 1.001
    assert c["host"]["cpu_model"] and c["host"]["threads_used"] >= 1
    # the passes one by one: each figure follows from its own time and its algorithmic bytes / flops
    p = b["passes"]
    n_m = p["shape"]["in_features"] * p["shape"]["hypercolumns"] * p["shape"]["minicolumns"]
    assert p["weight"]["hbm"]["algorithmic_bytes"] == 2 * 4 * n_m
    assert p["weight_masked"]["hbm"]["algorithmic_bytes"] == 2 * 4 * n_m + p["shape"]["in_features"] * p["shape"]["hypercolumns"]
    for name in ("trace", "weight", "weight_masked"):
        q = p[name]
        assert q["avg_us"] > 0
        assert q["hbm"]["GBps"] == pytest.approx(q["hbm"]["algorithmic_bytes"] / (q["avg_us"] * 1e-6) / 1e9, rel=1e-6)
        assert q["hbm"]["frac_of_hbm_peak"] == pytest.approx(q["hbm"]["GBps"] / 8000.0, rel=1e-9)
    for name in ("trace", "forward_dense"):
        q = p[name]
        assert q["mfma"]["flops"] == 2.0 * p["shape"]["batch"] * n_m
        assert 0.0 < q["mfma"]["frac_of_mfma_peak"] < 1.0
    o = b["other_configs"]["dense"]
    assert "configs[0]" in o["config"]["workload"] and o["value"] > 0 and 0.0 < o["roofline"]["frac"] < 1.0
    assert o["cpu_baseline"]["value"] > 0


def test_other_workload_line():
    b = _run("--workload", "dense", "--steps", "40", "--warmup", "10", "--no-cpu-baseline")
    assert b["n_gpus"] == 1 and b["dtype"] == "f32" and b["cpu_baseline"] is None
    assert b["roofline"]["bound"] in ("hbm", "mfma") and 0.0 < b["roofline"]["frac"] < 1.0
    assert "configs[0]" in b["config"]["workload"]
