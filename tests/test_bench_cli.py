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


def test_parity_outside_the_tolerance_sets_the_exit_status(oracle):
    """bench.py is a checker: a result outside the tolerance of the path is recorded and makes
    the run exit with a non-zero status (here: a scale wrong by 1 %)."""
    import importlib.util

    import numpy as np
    spec = importlib.util.spec_from_file_location("bench_under_test", BENCH)
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    rng = np.random.default_rng(5)
    K, N, q, g = 1024, 64, 3, 128
    bW = rng.integers(0, 2 ** 32, size=(K // 32, q, N), dtype=np.uint32)
    alpha = np.abs(rng.normal(0, 0.02, size=(K // g, q, N))).astype(np.float16)
    x = rng.normal(0, 1, size=(1, K)).astype(np.float16)
    truth = oracle.matvec_f64(bW, alpha, None, x)
    good = truth.astype(np.float16)
    rec = bench.parity_record(oracle, good, truth, N)
    assert rec["within_tolerance"] and rec["violation"] is None and bench.PARITY_FAILURES == []
    wrong = oracle.matvec_f64(bW, (alpha.astype(np.float32) * 1.01).astype(np.float16), None, x).astype(np.float16)
    rec = bench.parity_record(oracle, wrong, truth, N, label="scaled")
    assert not rec["within_tolerance"] and rec["violation"]
    assert len(bench.PARITY_FAILURES) == 1 and bench.PARITY_FAILURES[0].startswith("scaled: ")
