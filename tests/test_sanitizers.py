"""Host code under AddressSanitizer and UndefinedBehaviorSanitizer (no GPU, no HIP): the packer's
re-tiling and the CPU oracle, each driven over ragged shapes on exactly sized heap arrays, so that an
access outside an array or an overflowing index computation aborts the run.  The sanitizer run-time is
linked statically, so that libraries preloaded into the test process do not get in its way."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FLAGS = ["-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-static-libasan",
         "-static-libubsan"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
ENV.pop("LD_PRELOAD", None)


def build_and_run(tmp_path, compiler, sources, extra):
    exe = os.path.join(str(tmp_path), "sanitized")
    build = subprocess.run([compiler] + FLAGS + extra + sources + ["-o", exe, "-lpthread", "-lm"], capture_output=True, text=True)
    if build.returncode != 0 and ("libasan" in build.stderr or "libubsan" in build.stderr or "sanitize" in build.stderr):
        pytest.skip("this compiler has no sanitizer run-time: " + build.stderr.strip().splitlines()[-1])
    assert build.returncode == 0, build.stderr
    run = subprocess.run([exe], capture_output=True, text=True, env=ENV, timeout=300)
    assert run.returncode == 0, run.stdout + run.stderr
    return run.stdout


def test_packer_under_sanitizers(tmp_path):
    out = build_and_run(tmp_path, "g++", [os.path.join(ROOT, "tests", "cpp", "packer_sanitize.cpp"),
                                          os.path.join(ROOT, "lut-gemm_amd", "csrc", "packer.cpp")], ["-std=c++17"])
    assert "13 shapes ok" in out, out


def test_oracle_under_sanitizers(tmp_path):
    out = build_and_run(tmp_path, "gcc", [os.path.join(ROOT, "tests", "cpp", "oracle_sanitize.c"),
                                          os.path.join(ROOT, "oracle", "lutgemm_oracle.c")], ["-std=c11", "-fopenmp"])
    assert "oracle under sanitizers: ok" in out, out
