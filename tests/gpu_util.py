"""Helpers shared by the GPU parity tests: device buffers via torch (plumbing only), the
tolerance of the path, and a runner that calls the product through its C ABI binding."""
import numpy as np

# Tolerance of the path (fp16 in/out, fp32 accumulation, one final rounding), against the
# double-precision truth over the fp16-rounded inputs:
#   per element  |y - y*| <= 2 ulp_fp16(|y*|) + 1e-3      and      ||y - y*||2 / ||y*||2 <= 1e-3
ULPS = 2.0
ABS_TOL = 1e-3
REL_L2_TOL = 1e-3


def ulp_fp16(v):
    a = np.abs(np.asarray(v, np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -14)))
    return 2.0 ** (e - 10)


def assert_within_tolerance(y16, truth, what=""):
    y = np.asarray(y16, np.float16).astype(np.float64).reshape(-1)
    t = np.asarray(truth, np.float64).reshape(-1)
    assert np.all(np.isfinite(y)), what
    err = np.abs(y - t)
    bound = ULPS * ulp_fp16(t) + ABS_TOL
    worst = int(np.argmax(err - bound))
    assert np.all(err <= bound), "%s: element %d: got %r want %r err %g bound %g" % (
        what, worst, y[worst], t[worst], err[worst], bound[worst])
    den = np.linalg.norm(t)
    if den > 0:
        rel = np.linalg.norm(y - t) / den
        assert rel <= REL_L2_TOL, "%s: relative L2 error %g" % (what, rel)


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
