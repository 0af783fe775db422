"""The reference's C++ API (namespace lutGEMM: nQWeight_fp16, matmul, dequantize_*) as a header-only
layer over the C ABI: a caller in the reference's spelling (tests/cpp/dropin_test.cpp) compiles here,
and on the GPU reproduces the reference test's protocol with the numbers checked."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
BIN = os.path.join(CPP, "dropin_test")


def test_dropin_caller_compiles_against_public_headers(lutgemm):
    subprocess.run(["make", "-B", "-C", CPP], check=True, stdout=subprocess.DEVNULL)
    assert os.path.exists(BIN)
    # public data members keep the reference's names and order (nQWeight_fp16.h:29-37 of the reference)
    text = open(os.path.join(ROOT, "include", "nQWeight_fp16.h")).read()
    order = ["bWeight", "alpha", "q_bias", "num_groups", "group_size", "mSize", "kSize", "nb", "is_row_wise_quantize"]
    import re
    body = text[text.index("class nQWeight_fp16 {"):]
    body = body[:body.index("nQWeight_fp16() {}")]          # the data member declarations
    pos = [re.search(r"[ *]%s\b" % name, body).start() for name in order]
    assert pos == sorted(pos)


@pytest.mark.gpu
def test_dropin_caller_runs_reference_protocol(lutgemm):
    assert os.path.exists(BIN), "build the C++ test first (make -C tests/cpp, or __graft_entry__.build())"
    print("running", BIN, "full", flush=True)
    r = subprocess.run([BIN, "full"], capture_output=True, text=True, timeout=110)
    sys.stdout.write(r.stdout)
    sys.stderr.write(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "DROPIN OK" in r.stdout
    assert r.stdout.count("latency min") >= 6
