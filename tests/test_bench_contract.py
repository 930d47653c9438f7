"""CPU-side checks of bench.py's command line contract (nothing here touches a GPU)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True,
                          text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _bench("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_help_names_the_workloads():
    r = _bench("--help")
    assert r.returncode == 0
    for name in ("mnist", "dense", "wide64", "stl10", "largest", "--steps", "--warmup", "--gpus"):
        assert name in r.stdout


def test_trace_summary_reads_rocprofv3_kernel_stats(tmp_path):
    """`--trace-summary DIR`: the table kept under profiles/ from a kernel_stats.csv as rocprofv3 writes it."""
    d = tmp_path / "trace" / "host" / "1234"
    d.mkdir(parents=True)
    (d / "bench_kernel_stats.csv").write_text(
        '"Name","Calls","TotalDurationNs","AverageNs","Percentage","MinNs","MaxNs","StdDev"\n'
        '"void sb::k_train_fused<float, 32, true, 1, false, true>(sb::TrainArgs<float>)",4750,73720000,15520.0,57.66,11960,29160,900.1\n'
        '"__amd_rocclr_copyBuffer",480,2174400,4530.0,1.69,1200,6200,100.0\n')
    r = _bench("--trace-summary", str(tmp_path / "trace"))
    assert r.returncode == 0, r.stderr
    lines = r.stdout.splitlines()
    assert lines[0].split()[:2] == ["kernel", "calls"]
    assert lines[1].startswith("k_train_fused<float, 32, true, 1, false, true>")
    assert lines[1].split()[-5:] == ["4750", "15.52", "11.96", "29.16", "57.66"]
    assert lines[2].startswith("__amd_rocclr_copyBuffer")


def test_pmc_summary_scales_by_the_copy_calibration(tmp_path):
    """`--pmc-summary A,B --pmc-calibration C,D`: medians per kernel and counter, FETCH_SIZE / WRITE_SIZE scaled
    by what the same counters read for the 64 MiB copies, and the traffic line bench.py reads back."""
    def run(name, kernel, counter, values):
        d = tmp_path / name / "host" / "1"
        d.mkdir(parents=True)
        rows = ['"Dispatch_Id","Kernel_Name","Counter_Name","Counter_Value"']
        rows += [f'{i},"{kernel}","{counter}",{v}' for i, v in enumerate(values)]
        (d / "bench_counter_collection.csv").write_text("\n".join(rows) + "\n")
        return str(tmp_path / name)
    k = "void sb::k_train_fused<float, 32, true, 1, false, true>(sb::TrainArgs<float>)"
    fetch = run("fetch", k, "FETCH_SIZE", [14000.0, 14147.0, 15000.0])
    write = run("write", k, "WRITE_SIZE", [20310.0, 20310.0, 20311.0])
    cfetch = run("cfetch", "__amd_rocclr_copyBuffer", "FETCH_SIZE", [32768.0] * 3)  # reads half: scale 2
    cwrite = run("cwrite", "__amd_rocclr_copyBuffer", "WRITE_SIZE", [65536.0] * 3)
    r = _bench("--pmc-summary", f"{fetch},{write}", "--pmc-calibration", f"{cfetch},{cwrite}")
    assert r.returncode == 0, r.stderr
    out = r.stdout
    assert "kernel_source_stamp: " in out
    assert "scale 2.0000" in out and "scale 1.0000" in out
    assert "k_train_fused<float, 32, true, 1, false, true>" in out
    want = (14147.0 * 2 + 20310.0) * 1024
    line = [ln for ln in out.splitlines() if ln.startswith("traffic_bytes_per_launch:")]
    assert line and abs(float(line[0].split(":")[1]) - want) < 1.0


def test_bracket_calibration_leaves_carried_events_alone():
    """Kernels whose events ride on the launch keep their measured duration; the others lose the per-bracket
    cost that follows from the bracketed and the unbracketed pass, capped at an empty bracket's time."""
    sys.path.insert(0, ROOT)
    import bench
    kernels = {"train_fused": {"launches": 100, "raw_avg_us": 16.0, "events": "carried"},
               "forward": {"launches": 100, "raw_avg_us": 9.0, "events": "bracket"}}
    raw_ms = (100 * 16.0 + 100 * 9.0) / 1e3
    # unbracketed: 100 steps of 22.5 us -> the 100 brackets added 2.5 us each
    us = bench.calibrate_brackets(kernels, raw_ms, 100, 100 * 22.5e-6, upper_us=4.4)
    assert abs(us - 2.5) < 1e-9
    assert kernels["train_fused"]["avg_us"] == 16.0 and abs(kernels["forward"]["avg_us"] - 6.5) < 1e-9
    # a profiler that slows the bracketed pass down: no more than an empty bracket is taken off
    us = bench.calibrate_brackets(kernels, raw_ms + 1.0, 100, 100 * 22.5e-6, upper_us=4.4)
    assert us == 4.4 and abs(kernels["forward"]["avg_us"] - 4.6) < 1e-9
