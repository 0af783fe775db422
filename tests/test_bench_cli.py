"""bench.py's command line: the one-GPU guard and the option list (no GPU needed)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0
    assert "one GPU only" in r.stderr and "--gpus 2" in r.stderr
    assert r.stdout == ""  # no JSON line for a run that did not happen


def test_options():
    r = subprocess.run([sys.executable, BENCH, "--help"], capture_output=True, text=True)
    assert r.returncode == 0
    for opt in ("--gpus", "--steps", "--warmup", "--config", "--m", "--graph", "--plan", "--no-cpu", "--no-dense",
                "--copy-calibration"):
        assert opt in r.stdout
