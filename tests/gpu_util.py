"""Helpers shared by the GPU parity tests: device buffers via torch (plumbing only), the
tolerance of the path, and a runner that calls the product through its C ABI binding."""
import numpy as np

# The tolerance of the path is stated once, next to the oracle (oracle/oracle.py):
#   per element  |y - y*| <= 2 ulp_fp16(|y*|) + 1e-3      and      ||y - y*||2 / ||y*||2 <= 1e-3
from oracle.oracle import ABS_TOL, REL_L2_TOL, ULPS, tolerance_violation, ulp_fp16  # noqa: F401


def assert_within_tolerance(y16, truth, what=""):
    bad = tolerance_violation(y16, truth)
    assert bad is None, "%s: %s" % (what, bad)


def run_matvec(lg, weight, x16, device, cols=False):
    """x16: numpy float16 [m][k] -> numpy float16 [m][n] computed by the HIP library."""
    import torch
    x16 = np.ascontiguousarray(np.atleast_2d(x16), np.float16)
    m, k = x16.shape
    n = weight.mSize
    if cols:
        xd = torch.from_numpy(np.ascontiguousarray(x16.T)).to(device)
        yd = torch.full((n, m), float("nan"), dtype=torch.float16, device=device)
        weight.matvec_cols(xd.data_ptr(), yd.data_ptr(), m, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        return yd.cpu().numpy().T.copy()
    xd = torch.from_numpy(x16).to(device)
    yd = torch.full((m, n), float("nan"), dtype=torch.float16, device=device)
    weight.matvec(xd.data_ptr(), yd.data_ptr(), m, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    return yd.cpu().numpy()
