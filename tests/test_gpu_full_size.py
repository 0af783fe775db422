"""GPU parity at the benchmark's real shapes: cfg2 (k=12288, n=49152, q=4, offset), the sixteen
cfg3 points (k=n=7168) and the four cfg4 decoder-layer shapes with m in {1, 2, 4, 8} (FC2 has
k=49152 = 96 k-blocks, also run with 96 k-splits), and shapes at the ends of the range: one k-block
against 300,001 outputs, 256 k-blocks against 96 outputs or a single one.

The HIP path computes the whole problem.  Output columns are independent, so the oracle
(double accumulation over the fp16-rounded inputs) is evaluated on a strided subset of columns
plus the last ones, which keeps it to seconds; properties that need no oracle are checked over
the full width: a repeated launch is bit-identical, and a unit activation vector returns a row
of the dequantised weight bit for bit.  Tolerance of the floating-point path: gpu_util.py.
"""
import sys

import numpy as np
import pytest

from gpu_util import assert_within_tolerance, run_matvec

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def column_subset(n, count):
    """`count` columns spread over [0, n) with an odd stride, plus the first and last 40."""
    stride = max(1, (n // count) | 1)
    cols = np.concatenate([np.arange(0, n, stride)[:count], np.arange(min(40, n)), np.arange(max(0, n - 40), n)])
    return np.unique(cols)


def truth_on(oracle, w, x, cols):
    z = None
    if w["q_bias"] is not None:
        z = np.ascontiguousarray(w["q_bias"].astype(np.float16)[:, cols])
    return oracle.matvec_f64(np.ascontiguousarray(w["bW"][:, :, cols]),
                             np.ascontiguousarray(w["alpha"].astype(np.float16)[:, :, cols]), z, x)


def dense_rows_f16(oracle, w, rows, cols):
    """Rows `rows` of the dequantised weight (offset included) on columns `cols`, rounded once to
    fp16 from the exact sum."""
    z = None
    if w["q_bias"] is not None:
        z = np.ascontiguousarray(w["q_bias"].astype(np.float16)[:, cols])
    out = []
    for r in rows:
        w0 = r // 32
        g = w["g"]
        grp = r // g
        bW = np.ascontiguousarray(w["bW"][w0:w0 + 1][:, :, cols])
        alpha = np.ascontiguousarray(w["alpha"].astype(np.float16)[grp:grp + 1][:, :, cols])
        zz = None if z is None else np.ascontiguousarray(z[grp:grp + 1])
        dense = oracle.dense_weight_f64(bW, alpha, zz)          # 32 rows of this word
        out.append(dense[r % 32].astype(np.float16))
    return np.stack(out)


def check_full(lg, oracle, device, w, W, x, cols, what):
    y = run_matvec(lg, W, x, device)
    assert y.shape == (x.shape[0], w["n"])
    assert_within_tolerance(y[:, cols], truth_on(oracle, w, x, cols), what)
    y2 = run_matvec(lg, W, x, device)
    assert np.array_equal(y.view(np.uint16), y2.view(np.uint16)), what + ": repeat differs"
    return y


def check_unit_rows(lg, oracle, device, w, W, rows, cols, what):
    for r in rows:
        e = np.zeros((1, w["k"]), np.float16)
        e[0, r] = 1
        ye = run_matvec(lg, W, e, device)
        want = dense_rows_f16(oracle, w, [r], cols)[0]
        assert np.array_equal(ye[0, cols].view(np.uint16), want.view(np.uint16)), "%s: unit row %d" % (what, r)


def test_cfg2_full_size(lutgemm, oracle, device):
    from lutgemm import synth
    c = synth.CONFIGS["cfg2"]
    k, n, q, g = c["k"], c["n"], c["q"], c["g"]
    say("case cfg2 full", k, n, q, g)
    w = synth.make_weight(k, n, q, g, rtn=True, seed=2)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    x = synth.make_x(1, k, seed=2)
    cols = column_subset(n, 1500)
    check_full(lutgemm, oracle, device, w, W, x, cols, "cfg2 plan=%s" % W.plan())
    check_unit_rows(lutgemm, oracle, device, w, W, [0, 5000, k - 1], cols, "cfg2")
    # a second plan with more k-splits than the automatic one
    W.set_plan(6, 12)
    check_full(lutgemm, oracle, device, w, W, x, cols, "cfg2 plan=%s" % W.plan())
    W.close()


@pytest.mark.parametrize("q", [1, 2, 3, 4])
@pytest.mark.parametrize("g", [32, 64, 128, 7168])
def test_cfg3_full_size(lutgemm, oracle, device, q, g):
    from lutgemm import synth
    k = n = 7168
    say("case cfg3 full", q, g)
    w = synth.make_weight(k, n, q, g, seed=q * 10000 + g)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, None)
    x = synth.make_x(1, k, seed=q + g)
    cols = column_subset(n, 1024)
    check_full(lutgemm, oracle, device, w, W, x, cols, "cfg3 q=%d g=%d plan=%s" % (q, g, W.plan()))
    check_unit_rows(lutgemm, oracle, device, w, W, [g - 1, k - 1], cols, "cfg3 q=%d g=%d" % (q, g))
    W.close()


@pytest.mark.parametrize("layer", ["qkv", "out", "fc1", "fc2"])
def test_cfg4_full_size_all_batches(lutgemm, oracle, device, layer):
    from lutgemm import synth
    L = synth.CFG4_LAYERS[layer]
    k, n, q, g = L["k"], L["n"], 2, 128
    say("case cfg4 full", layer, k, n)
    w = synth.make_weight(k, n, q, g, seed=400 + len(layer) + k // 1024)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, None)
    cols = column_subset(n, 768)
    plans = [(0, 0)]
    if layer == "fc2":
        plans.append((4, 96))     # one k-block per workgroup: 96 k-splits
    for waves, ks in plans:
        W.set_plan(waves, ks)
        rows_m1 = None
        for m in (1, 2, 4, 8):
            say("case cfg4 full", layer, "m", m, "plan", W.plan())
            x = synth.make_x(8, k, seed=77)[:m]
            y = check_full(lutgemm, oracle, device, w, W, x, cols, "cfg4 %s m=%d plan=%s" % (layer, m, W.plan()))
            if m == 1:
                rows_m1 = y
        assert rows_m1 is not None
    check_unit_rows(lutgemm, oracle, device, w, W, [k - 1], cols, "cfg4 %s" % layer)
    W.close()


@pytest.mark.parametrize("k,n,q,g,offset", [
    (32, 300001, 3, 32, True),        # a single ragged k-block, 9,376 output batches
    (131072, 96, 8, 128, False),      # 256 k-blocks, three output batches, eight planes
    (98304, 1, 2, 64, True),          # a single output
    (64, 70000, 8, 64, True),
])
def test_extreme_aspect_ratios(lutgemm, oracle, device, k, n, q, g, offset):
    """Very wide and very deep weights, every kernel family (one row, two rows, the batch kernel in
    one and in two passes), rows and columns entry; the whole output is compared with the oracle."""
    from lutgemm import synth
    w = synth.make_weight(k, n, q, g, offset=offset, seed=k % 1000 + n % 1000)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    cols = np.arange(n)
    for m in (1, 2, 5, 19):
        say("case extreme", k, n, q, g, offset, "m", m, W.plan(m))
        x = synth.make_x(m, k, seed=m)
        truth = truth_on(oracle, w, x, cols)
        for by_cols in (False, True):
            y = run_matvec(lutgemm, W, x, device, cols=by_cols)
            assert_within_tolerance(y, truth, "k=%d n=%d q=%d m=%d cols=%s" % (k, n, q, m, by_cols))
    W.close()
