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
