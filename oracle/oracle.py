"""ctypes/numpy front end of the CPU oracle (liblutgemm_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  The product library never imports this module.

Array conventions are those of lutgemm_oracle.c: bW uint32 [K/32][q][N], alpha/zoff as
numpy float16 [G][q][N] / [G][N], x float16 [M][K].
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liblutgemm_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (make -B when force)."""
    cmd = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        vp, i, l = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
        L.orc_h2f.restype = ctypes.c_float
        L.orc_h2f.argtypes = [ctypes.c_uint16]
        L.orc_f2h.restype = ctypes.c_uint16
        L.orc_f2h.argtypes = [ctypes.c_float]
        L.orc_d2h.restype = ctypes.c_uint16
        L.orc_d2h.argtypes = [ctypes.c_double]
        for name in ("orc_f2h_array", "orc_d2h_array", "orc_h2f_array"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [vp, vp, l]
        L.orc_pack_signs.restype = None
        L.orc_pack_signs.argtypes = [vp, vp, i, i, i]
        L.orc_dequantize_cpu.restype = None
        L.orc_dequantize_cpu.argtypes = [vp, vp, i, i, i, i, i, vp]
        L.orc_dequantize_cpu_omp.restype = i
        L.orc_dequantize_cpu_omp.argtypes = [vp, vp, i, i, i, i, vp]
        L.orc_dense_weight_f64.restype = None
        L.orc_dense_weight_f64.argtypes = [vp, vp, vp, i, i, i, i, vp]
        L.orc_matmul_cpu.restype = None
        L.orc_matmul_cpu.argtypes = [vp, vp, i, i, i, vp]
        L.orc_matmul_cpu_omp.restype = i
        L.orc_matmul_cpu_omp.argtypes = [vp, vp, i, i, i, vp]
        L.orc_matvec_f64.restype = None
        L.orc_matvec_f64.argtypes = [vp, vp, vp, vp, i, i, i, i, i, vp]
        L.orc_lut256_f64.restype = None
        L.orc_lut256_f64.argtypes = [vp, vp]
        L.orc_ref_kernel_fp16.restype = None
        L.orc_ref_kernel_fp16.argtypes = [vp, vp, vp, vp, i, i, i, i, i, vp]
        L.orc_rtn_to_bcq.restype = None
        L.orc_rtn_to_bcq.argtypes = [vp, vp, vp, i, i, i, i, vp, vp, vp]
        L.orc_error_stats.restype = None
        L.orc_error_stats.argtypes = [vp, vp, l, vp]
        _lib = L
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def f2h(a):
    """float32 array -> binary16 bit patterns (uint16), RNE, bit routine."""
    a = _c(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f2h_array(_p(a), _p(out), a.size)
    return out


def d2h(a):
    """float64 array -> binary16 bit patterns (uint16), RNE, definition routine."""
    a = _c(a, np.float64)
    out = np.empty(a.shape, np.uint16)
    lib().orc_d2h_array(_p(a), _p(out), a.size)
    return out


def h2f(a):
    a = _c(a, np.uint16)
    out = np.empty(a.shape, np.float32)
    lib().orc_h2f_array(_p(a), _p(out), a.size)
    return out


def pack_signs(signs):
    """signs int8 [K][q][N] of +/-1 -> bW uint32 [K/32][q][N]."""
    signs = _c(signs, np.int8)
    K, q, N = signs.shape
    bW = np.empty((K // 32, q, N), np.uint32)
    lib().orc_pack_signs(_p(signs), _p(bW), K, q, N)
    return bW


def _dims(bW, alpha):
    KW, q, N = bW.shape
    G = alpha.shape[0]
    K = KW * 32
    return K, N, q, G, K // G


def dequantize_cpu(bW, alpha, row_wise=False):
    """Reference CPU dequantisation (offset ignored, as the reference does): fp16 [K][N]
    (or [N][K] when row_wise)."""
    bW = _c(bW, np.uint32)
    alpha = _c(alpha, np.float16)
    K, N, q, G, gs = _dims(bW, alpha)
    fW = np.empty((N, K) if row_wise else (K, N), np.float16)
    lib().orc_dequantize_cpu(_p(bW), _p(alpha), K, N, q, gs, int(row_wise), _p(fW))
    return fW


def dequantize_cpu_omp(bW, alpha):
    bW = _c(bW, np.uint32)
    alpha = _c(alpha, np.float16)
    K, N, q, G, gs = _dims(bW, alpha)
    fW = np.empty((K, N), np.float16)
    used = lib().orc_dequantize_cpu_omp(_p(bW), _p(alpha), K, N, q, gs, _p(fW))
    return fW, used


def dense_weight_f64(bW, alpha, zoff=None):
    bW = _c(bW, np.uint32)
    alpha = _c(alpha, np.float16)
    zoff = _c(zoff, np.float16) if zoff is not None else None
    K, N, q, G, gs = _dims(bW, alpha)
    W = np.empty((K, N), np.float64)
    lib().orc_dense_weight_f64(_p(bW), _p(alpha), _p(zoff), K, N, q, gs, _p(W))
    return W


def matmul_cpu(x, fW):
    """Reference float triple loop: x fp16 [M][K], fW fp16 [K][N] -> float32 [M][N]."""
    x = _c(np.atleast_2d(x), np.float16)
    fW = _c(fW, np.float16)
    M, K = x.shape
    N = fW.shape[1]
    out = np.empty((M, N), np.float32)
    lib().orc_matmul_cpu(_p(x), _p(fW), M, N, K, _p(out))
    return out


def matmul_cpu_omp(x, fW):
    x = _c(np.atleast_2d(x), np.float16)
    fW = _c(fW, np.float16)
    M, K = x.shape
    N = fW.shape[1]
    out = np.empty((M, N), np.float32)
    used = lib().orc_matmul_cpu_omp(_p(x), _p(fW), M, N, K, _p(out))
    return out, used


def matvec_f64(bW, alpha, zoff, x):
    """Double-precision truth y[M][N] over the fp16-rounded inputs."""
    bW = _c(bW, np.uint32)
    alpha = _c(alpha, np.float16)
    zoff = _c(zoff, np.float16) if zoff is not None else None
    x = _c(np.atleast_2d(x), np.float16)
    K, N, q, G, gs = _dims(bW, alpha)
    M = x.shape[0]
    assert x.shape[1] == K
    y = np.empty((M, N), np.float64)
    lib().orc_matvec_f64(_p(bW), _p(alpha), _p(zoff), _p(x), M, K, N, q, gs, _p(y))
    return y


def lut256_f64(x8):
    x8 = _c(x8, np.float16)
    assert x8.size == 8
    out = np.empty(256, np.float64)
    lib().orc_lut256_f64(_p(x8), _p(out))
    return out


def ref_kernel_fp16(bW, alpha, zoff, x, fused=True):
    """fp16 emulation of the reference GPU kernel for one activation vector -> fp16 [N]."""
    bW = _c(bW, np.uint32)
    alpha = _c(alpha, np.float16)
    zoff = _c(zoff, np.float16) if zoff is not None else None
    x = _c(x, np.float16).reshape(-1)
    K, N, q, G, gs = _dims(bW, alpha)
    y = np.empty(N, np.float16)
    lib().orc_ref_kernel_fp16(_p(bW), _p(alpha), _p(zoff), _p(x), K, N, q, gs, int(fused), _p(y))
    return y


def rtn_to_bcq(codes, scale, zero, q, group_size):
    """codes uint8 [K][N], scale/zero float32 [G][N] -> (bW, alpha float32 [G][q][N], off [G][N])."""
    codes = _c(codes, np.uint8)
    scale = _c(scale, np.float32)
    zero = _c(zero, np.float32)
    K, N = codes.shape
    G = K // group_size
    bW = np.empty((K // 32, q, N), np.uint32)
    alpha = np.empty((G, q, N), np.float32)
    off = np.empty((G, N), np.float32)
    lib().orc_rtn_to_bcq(_p(codes), _p(scale), _p(zero), K, N, q, group_size, _p(bW), _p(alpha), _p(off))
    return bW, alpha, off


def error_stats(y_h, truth):
    """(mean abs, max abs, relative L2) of an fp16 result against a float64 truth."""
    y_h = _c(y_h, np.float16).reshape(-1)
    truth = _c(truth, np.float64).reshape(-1)
    out = np.zeros(3, np.float64)
    lib().orc_error_stats(_p(y_h), _p(truth), y_h.size, _p(out))
    return tuple(out)


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


def tolerance_violation(y16, truth):
    """None if the fp16 result is within the tolerance above of the float64 truth, else a
    description of the worst violation."""
    y = np.asarray(y16, np.float16).astype(np.float64).reshape(-1)
    t = np.asarray(truth, np.float64).reshape(-1)
    if y.shape != t.shape:
        return "shape mismatch: %r against %r" % (y.shape, t.shape)
    if not np.all(np.isfinite(y)):
        return "%d non-finite outputs" % int((~np.isfinite(y)).sum())
    err = np.abs(y - t)
    bound = ULPS * ulp_fp16(t) + ABS_TOL
    if not np.all(err <= bound):
        worst = int(np.argmax(err - bound))
        return "element %d: got %r want %r err %g bound %g" % (worst, y[worst], t[worst], err[worst], bound[worst])
    den = np.linalg.norm(t)
    if den > 0:
        rel = np.linalg.norm(y - t) / den
        if rel > REL_L2_TOL:
            return "relative L2 error %g above %g" % (rel, REL_L2_TOL)
    return None
