"""The allocation-free entry point lutgemm_matvec_static (split-k words in a static device array)
against lutgemm_matvec on the same inputs, through the C ABI: bit for bit, on calls in a row
(three, two, one and nine activation rows: batch, two-row and one-row kernels), the second on a
smaller weight than the first, so that words left behind by a call would show in the next."""
import ctypes
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def run(lg, W, x16, device, static):
    import torch
    m, k = x16.shape
    xd = torch.from_numpy(np.ascontiguousarray(x16)).to(device)
    yd = torch.full((m, W.mSize), float("nan"), dtype=torch.float16, device=device)
    fn = lg.load().lutgemm_matvec_static if static else lg.load().lutgemm_matvec
    st = fn(W._h, ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(yd.data_ptr()), m,
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert st == 0, lg.load().lutgemm_last_error().decode()
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def test_static_workspace_entry_point_matches_matvec(lutgemm, oracle, device):
    from lutgemm import synth
    from gpu_util import assert_within_tolerance
    # first call: k-splits over a wide weight; second call: a smaller weight with other splits
    for (k, n, q, g, off, plan, m) in [(8192, 6000, 3, 128, True, (8, 8), 3), (2048, 1000, 2, 64, False, (3, 4), 2),
                                        (4096, 4096, 3, 128, False, (0, 0), 1), (4096, 2080, 2, 128, False, (0, 0), 9)]:
        print("case static", k, n, q, g, off, plan, m, flush=True)
        sys.stdout.flush()
        w = synth.make_weight(k, n, q, g, offset=off, seed=k + n)
        W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
        W.set_plan(*plan)
        x = synth.make_x(m, k, seed=n)
        want = run(lutgemm, W, x, device, static=False)
        got = run(lutgemm, W, x, device, static=True)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
        again = run(lutgemm, W, x, device, static=True)
        assert np.array_equal(again.view(np.uint16), want.view(np.uint16))
        z = w["q_bias"].astype(np.float16) if off else None
        assert_within_tolerance(got, oracle.matvec_f64(w["bW"], w["alpha"].astype(np.float16), z, x), "static")
        W.close()


def test_static_workspace_rejects_what_it_cannot_hold(lutgemm, device):
    from lutgemm import synth
    import torch
    L = lutgemm.load()
    k, n = 32, 65536 + 32
    w = synth.make_weight(k, n, 1, 32, seed=1)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, 1, 1, None)
    xd = torch.zeros((1, k), dtype=torch.float16, device=device)
    yd = torch.zeros((1, n), dtype=torch.float16, device=device)
    st = L.lutgemm_matvec_static(W._h, ctypes.c_void_p(xd.data_ptr()), ctypes.c_void_p(yd.data_ptr()), 1, None)
    assert st == lutgemm.ERR_UNSUPPORTED
    assert b"static workspace" in L.lutgemm_last_error()
    W.close()
