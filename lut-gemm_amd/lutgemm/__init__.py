"""ctypes binding of liblutgemm_hip.so (the C ABI in include/lutgemm_c.h).

Mirrors the reference's C++ surface for the BCQ matvec path:
  BCQWeight(bW, alpha, k, n, q, num_groups, q_bias)  ~ lutGEMM::nQWeight_fp16::parsing
                                                      (lutGEMM/src/nQWeight_fp16.cu:60-91)
  matmul(output, input, weight, m)                   ~ lutGEMM::matmul(void*, void*, nQWeight_fp16&, int)
                                                      (lutGEMM/src/kernels.cu:64-71)
Device buffers are passed as integer addresses (e.g. torch.Tensor.data_ptr()); torch is only
plumbing for device memory and streams (it is imported, when present, solely so that both
share one HIP runtime).

There is no CPU fallback: if the HIP library is missing, loading raises.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "liblutgemm_hip.so")

OK = 0
ERR_NULL_POINTER, ERR_BAD_SHAPE, ERR_NO_DEVICE, ERR_HIP, ERR_OUT_OF_MEMORY, ERR_UNSUPPORTED, ERR_IO = range(1, 8)
MAX_BATCH = 4096

# every symbol include/lutgemm_c.h declares
EXPORTED = [
    "lutgemm_weight_create", "lutgemm_weight_create_f16", "lutgemm_weight_destroy", "lutgemm_weight_info",
    "lutgemm_matvec", "lutgemm_matvec_cols", "lutgemm_matvec_many", "lutgemm_dequantize", "lutgemm_weight_unpack",
    "lutgemm_weight_plan", "lutgemm_weight_plan_for", "lutgemm_weight_set_plan", "lutgemm_weight_set_batch_plan", "lutgemm_weight_autotune", "lutgemm_weight_device_ptrs", "lutgemm_packed_sizes",
    "lutgemm_pack_host", "lutgemm_unpack_host", "lutgemm_float_to_half", "lutgemm_last_error",
    "lutgemm_status_string", "lutgemm_version", "lutgemm_pack_file", "lutgemm_unpack_file", "lutgemm_weight_save",
    "lutgemm_weight_load", "lutgemm_weight_clone", "lutgemm_read_probe", "lutgemm_dense_gemv_f16",
    "lutgemm_weight_reset_workspace", "lutgemm_matvec_static", "lutgemm_matvec_each",
    "lutgemm_matvec_many_autotune", "lutgemm_matvec_many_plan",
]


class LutGemmError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("lutgemm status %d: %s" % (status, message))
        self.status = status


class WeightInfo(ctypes.Structure):
    _fields_ = [("k", ctypes.c_int), ("n", ctypes.c_int), ("q", ctypes.c_int), ("num_groups", ctypes.c_int),
                ("group_size", ctypes.c_int), ("has_offset", ctypes.c_int), ("sign_bytes", ctypes.c_size_t),
                ("scale_bytes", ctypes.c_size_t), ("offset_bytes", ctypes.c_size_t),
                ("device_bytes", ctypes.c_size_t)]


_lib = None


def load():
    """Load liblutgemm_hip.so; raises if it has not been built (no fallback)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise FileNotFoundError(
            "%s is missing: build it with `make -C %s` (or __graft_entry__.build())"
            % (LIB_PATH, os.path.join(os.path.dirname(_HERE), "csrc")))
    # One process must use one HIP runtime.  PyTorch-ROCm ships its own libamdhip64 with the
    # same soname as the system one; importing torch first makes this library bind to the copy
    # torch uses, so device pointers and streams made by torch are valid here.  Without torch the
    # system runtime is used.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = ctypes.CDLL(LIB_PATH)
    vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    pp = ctypes.POINTER(ctypes.c_void_p)
    pi = ctypes.POINTER(ctypes.c_int)
    psz = ctypes.POINTER(ctypes.c_size_t)
    L.lutgemm_weight_create.argtypes = [vp, vp, vp, i, i, i, i, pp]
    L.lutgemm_weight_create_f16.argtypes = [vp, vp, vp, i, i, i, i, pp]
    L.lutgemm_weight_destroy.argtypes = [vp]
    L.lutgemm_weight_info.argtypes = [vp, ctypes.POINTER(WeightInfo)]
    L.lutgemm_matvec.argtypes = [vp, vp, vp, i, vp]
    L.lutgemm_matvec_cols.argtypes = [vp, vp, vp, i, vp]
    L.lutgemm_matvec_static.argtypes = [vp, vp, vp, i, vp]
    L.lutgemm_matvec_many.argtypes = [vp, vp, vp, vp, i, vp]
    L.lutgemm_matvec_each.argtypes = [vp, vp, vp, vp, i, vp]
    L.lutgemm_matvec_many_autotune.argtypes = [vp, vp, vp, vp, i, vp]
    L.lutgemm_matvec_many_plan.argtypes = [vp, vp, vp, vp, i, pi, pi, pi, pi]
    L.lutgemm_dequantize.argtypes = [vp, vp, i, vp]
    L.lutgemm_weight_unpack.argtypes = [vp, vp, vp, vp]
    L.lutgemm_weight_plan.argtypes = [vp, pi, pi, pi, pi]
    L.lutgemm_weight_plan_for.argtypes = [vp, ctypes.c_int, pi, pi, pi, pi]
    L.lutgemm_weight_set_batch_plan.argtypes = [vp, ctypes.c_int, ctypes.c_int]
    L.lutgemm_pack_file.argtypes = [vp, vp, vp, i, i, i, i, ctypes.c_char_p]
    L.lutgemm_unpack_file.argtypes = [ctypes.c_char_p, vp, vp, vp, ctypes.POINTER(WeightInfo)]
    L.lutgemm_weight_save.argtypes = [vp, ctypes.c_char_p]
    L.lutgemm_weight_load.argtypes = [ctypes.c_char_p, pp]
    L.lutgemm_weight_clone.argtypes = [vp, pp]
    L.lutgemm_read_probe.argtypes = [vp, i, vp]
    L.lutgemm_dense_gemv_f16.argtypes = [vp, vp, vp, i, i, vp]
    L.lutgemm_weight_set_plan.argtypes = [vp, i, i]
    L.lutgemm_weight_reset_workspace.argtypes = [vp, vp]
    L.lutgemm_weight_autotune.argtypes = [vp, vp]
    L.lutgemm_weight_device_ptrs.argtypes = [vp, pp, pp, pp]
    L.lutgemm_packed_sizes.argtypes = [i, i, i, i, i, psz, psz]
    L.lutgemm_pack_host.argtypes = [vp, vp, vp, i, i, i, i, vp, vp]
    L.lutgemm_unpack_host.argtypes = [vp, vp, i, i, i, i, i, vp, vp, vp]
    L.lutgemm_float_to_half.argtypes = [vp, vp, sz]
    for name in EXPORTED:
        getattr(L, name).restype = ctypes.c_int
    L.lutgemm_last_error.restype = ctypes.c_char_p
    L.lutgemm_last_error.argtypes = []
    L.lutgemm_status_string.restype = ctypes.c_char_p
    L.lutgemm_status_string.argtypes = [i]
    L.lutgemm_version.restype = ctypes.c_char_p
    L.lutgemm_version.argtypes = []
    _lib = L
    return L


def _check(status):
    if status != OK:
        raise LutGemmError(status, load().lutgemm_last_error().decode())


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def float_to_half_bits(a):
    """float32 -> binary16 bit patterns with the library's ingest rounding."""
    a = np.ascontiguousarray(a, np.float32)
    out = np.empty(a.shape, np.uint16)
    _check(load().lutgemm_float_to_half(_ptr(a), _ptr(out), a.size))
    return out


def packed_sizes(k, n, q, num_groups, has_offset):
    s, c = ctypes.c_size_t(), ctypes.c_size_t()
    _check(load().lutgemm_packed_sizes(k, n, q, num_groups, int(has_offset), ctypes.byref(s), ctypes.byref(c)))
    return s.value, c.value


def pack_host(bW, alpha_h, q_bias_h, k, n, q, num_groups):
    """Host re-tiling: (bW uint32 [k/32][q][n], alpha uint16 [G][q][n], q_bias uint16 [G][n]|None)
    -> (sign tiles uint8, scale tiles uint16)."""
    bW = np.ascontiguousarray(bW, np.uint32)
    alpha_h = np.ascontiguousarray(alpha_h, np.uint16)
    q_bias_h = np.ascontiguousarray(q_bias_h, np.uint16) if q_bias_h is not None else None
    sb, cb = packed_sizes(k, n, q, num_groups, q_bias_h is not None)
    signs = np.empty(sb, np.uint8)
    scales = np.empty(cb // 2, np.uint16)
    _check(load().lutgemm_pack_host(_ptr(bW), _ptr(alpha_h), _ptr(q_bias_h), k, n, q, num_groups,
                                    _ptr(signs), _ptr(scales)))
    return signs, scales


def unpack_host(signs, scales, k, n, q, num_groups, has_offset):
    bW = np.empty((k // 32, q, n), np.uint32)
    alpha = np.empty((num_groups, q, n), np.uint16)
    q_bias = np.empty((num_groups, n), np.uint16) if has_offset else None
    _check(load().lutgemm_unpack_host(_ptr(signs), _ptr(scales), k, n, q, num_groups, int(has_offset),
                                      _ptr(bW), _ptr(alpha), _ptr(q_bias)))
    return bW, alpha, q_bias


def pack_file(path, bW, alpha, k, n, q, num_groups=1, q_bias=None):
    """Host only: write a packed-weight file from arrays in the reference layout."""
    bW = np.ascontiguousarray(bW, np.uint32)
    a = float_to_half_bits(alpha) if np.asarray(alpha).dtype != np.float16 else np.ascontiguousarray(alpha).view(np.uint16)
    z = None
    if q_bias is not None:
        z = float_to_half_bits(q_bias) if np.asarray(q_bias).dtype != np.float16 else np.ascontiguousarray(q_bias).view(np.uint16)
    if bW.size != (k // 32) * q * n or a.size != num_groups * q * n or (z is not None and z.size != num_groups * n):
        raise LutGemmError(ERR_BAD_SHAPE, "array sizes do not match k=%d n=%d q=%d num_groups=%d" % (k, n, q, num_groups))
    _check(load().lutgemm_pack_file(_ptr(bW), _ptr(a), _ptr(z), k, n, q, num_groups, os.fsencode(path)))


def unpack_file(path):
    """Host only: packed-weight file -> dict(bW uint32, alpha float16, q_bias float16|None, k, n, q, num_groups)."""
    info = WeightInfo()
    _check(load().lutgemm_unpack_file(os.fsencode(path), None, None, None, ctypes.byref(info)))
    bW = np.empty((info.k // 32, info.q, info.n), np.uint32)
    alpha = np.empty((info.num_groups, info.q, info.n), np.uint16)
    q_bias = np.empty((info.num_groups, info.n), np.uint16) if info.has_offset else None
    _check(load().lutgemm_unpack_file(os.fsencode(path), _ptr(bW), _ptr(alpha), _ptr(q_bias), None))
    return dict(bW=bW, alpha=alpha.view(np.float16), q_bias=q_bias.view(np.float16) if q_bias is not None else None,
                k=info.k, n=info.n, q=info.q, num_groups=info.num_groups)


class BCQWeight:
    """Packed BCQ weight on the current HIP device (the nQWeight_fp16 of this library).

    bW uint32 [k/32][q][n]; alpha float32 (or float16) [num_groups][q][n]; q_bias likewise
    [num_groups][n] or None.  Field names follow nQWeight_fp16: kSize, mSize, nb, num_groups,
    group_size (lutGEMM/include/nQWeight_fp16.h:29-37).
    """

    def __init__(self, bW, alpha, k, n, q, num_groups=1, q_bias=None):
        L = load()
        self._h = ctypes.c_void_p()
        bW = np.ascontiguousarray(bW, np.uint32)
        if bW.size != (k // 32) * q * n:
            raise LutGemmError(ERR_BAD_SHAPE, "bW has %d words, expected %d" % (bW.size, (k // 32) * q * n))
        alpha = np.asarray(alpha)
        if alpha.size != num_groups * q * n:
            raise LutGemmError(ERR_BAD_SHAPE, "alpha has %d entries, expected %d" % (alpha.size, num_groups * q * n))
        if q_bias is not None and np.asarray(q_bias).size != num_groups * n:
            raise LutGemmError(ERR_BAD_SHAPE, "q_bias has %d entries, expected %d" % (np.asarray(q_bias).size, num_groups * n))
        if alpha.dtype == np.float16:
            a = np.ascontiguousarray(alpha).view(np.uint16)
            z = np.ascontiguousarray(q_bias, np.float16).view(np.uint16) if q_bias is not None else None
            st = L.lutgemm_weight_create_f16(_ptr(bW), _ptr(a), _ptr(z), k, n, q, num_groups, ctypes.byref(self._h))
        else:
            a = np.ascontiguousarray(alpha, np.float32)
            z = np.ascontiguousarray(q_bias, np.float32) if q_bias is not None else None
            st = L.lutgemm_weight_create(_ptr(bW), _ptr(a), _ptr(z), k, n, q, num_groups, ctypes.byref(self._h))
        _check(st)
        self._read_info()

    def _read_info(self):
        info = self.info()
        self.kSize, self.mSize, self.nb = info.k, info.n, info.q
        self.num_groups, self.group_size = info.num_groups, info.group_size
        self.has_offset = bool(info.has_offset)

    @classmethod
    def _from_handle(cls, handle):
        self = cls.__new__(cls)
        self._h = handle
        self._read_info()
        return self

    @classmethod
    def load(cls, path):
        """Handle on the current device from a packed-weight file (no packing work)."""
        h = ctypes.c_void_p()
        _check(load().lutgemm_weight_load(os.fsencode(path), ctypes.byref(h)))
        return cls._from_handle(h)

    def save(self, path):
        _check(load().lutgemm_weight_save(self._h, os.fsencode(path)))

    def clone(self):
        """Independent handle with its own device copy and workspace, same launch plan."""
        h = ctypes.c_void_p()
        _check(load().lutgemm_weight_clone(self._h, ctypes.byref(h)))
        return BCQWeight._from_handle(h)

    def info(self):
        info = WeightInfo()
        _check(load().lutgemm_weight_info(self._h, ctypes.byref(info)))
        return info

    def plan(self, m=1):
        """Launch plan of calls with m activation rows (one-row, two-row or batch kernel)."""
        v = [ctypes.c_int() for _ in range(4)]
        _check(load().lutgemm_weight_plan_for(self._h, m, *[ctypes.byref(x) for x in v]))
        return dict(workgroups=v[0].value, waves=v[1].value, k_splits=v[2].value, k_blocks=v[3].value)

    def set_plan(self, waves=0, k_splits=0):
        _check(load().lutgemm_weight_set_plan(self._h, waves, k_splits))

    def set_batch_plan(self, waves=0, k_splits=0):
        """Launch plan of the batch kernel (3 or more rows); defaults: back to the automatic choice."""
        _check(load().lutgemm_weight_set_batch_plan(self._h, waves, k_splits))

    def autotune(self, stream=0):
        """Measure candidate launch plans on the device and keep the fastest; returns the plan."""
        _check(load().lutgemm_weight_autotune(self._h, stream or None))
        return self.plan()

    def reset_workspace(self, stream=0):
        """Zero the split-k accumulators and release the per-stream sets (only needed after an
        aborted launch)."""
        _check(load().lutgemm_weight_reset_workspace(self._h, stream or None))

    def weight_bytes(self):
        """Algorithmic packed-weight bytes: signs + scales + offsets (unpadded)."""
        i = self.info()
        return i.sign_bytes + i.scale_bytes + i.offset_bytes

    def matvec(self, x_ptr, y_ptr, m=1, stream=0):
        _check(load().lutgemm_matvec(self._h, x_ptr, y_ptr, m, stream or None))

    def matvec_static(self, x_ptr, y_ptr, m=1, stream=0):
        """matvec with the split-k words in the library's static device array: allocates nothing."""
        _check(load().lutgemm_matvec_static(self._h, x_ptr, y_ptr, m, stream or None))

    def matvec_cols(self, x_ptr, y_ptr, m=1, stream=0):
        _check(load().lutgemm_matvec_cols(self._h, x_ptr, y_ptr, m, stream or None))

    def dequantize(self, out_ptr, transposed=False, stream=0):
        _check(load().lutgemm_dequantize(self._h, out_ptr, int(transposed), stream or None))

    def unpack(self):
        i = self.info()
        bW = np.empty((i.k // 32, i.q, i.n), np.uint32)
        alpha = np.empty((i.num_groups, i.q, i.n), np.uint16)
        z = np.empty((i.num_groups, i.n), np.uint16) if i.has_offset else None
        _check(load().lutgemm_weight_unpack(self._h, _ptr(bW), _ptr(alpha), _ptr(z)))
        return bW, alpha.view(np.float16), (z.view(np.float16) if z is not None else None)

    def close(self):
        if self._h:
            load().lutgemm_weight_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def matmul(output_ptr, input_ptr, weight, m=1, stream=0):
    """lutGEMM::matmul(output, input, nqW, m): y[m][n] = x[m][k] * W."""
    weight.matvec(input_ptr, output_ptr, m, stream)


class MatvecSequence:
    """A fixed list of (weight, x_ptr, y_ptr, m) issued with one lutgemm_matvec_many call
    (independent neighbours share launches) or, with fused=False, one lutgemm_matvec_each call
    (one launch per entry)."""

    def __init__(self, items):
        n = len(items)
        self._keep = [it[0] for it in items]
        self.count = n
        self._ws = (ctypes.c_void_p * n)(*[it[0]._h for it in items])
        self._xs = (ctypes.c_void_p * n)(*[it[1] for it in items])
        self._ys = (ctypes.c_void_p * n)(*[it[2] for it in items])
        self._ms = (ctypes.c_int * n)(*[it[3] for it in items])

    def launch(self, stream=0, fused=True):
        fn = load().lutgemm_matvec_many if fused else load().lutgemm_matvec_each
        _check(fn(self._ws, self._xs, self._ys, self._ms, self.count, stream or None))

    def autotune(self, stream=0):
        """Measure the launch shapes of the fused launches of this list and remember the fastest for
        every list of the same shapes (lutgemm_matvec_many_autotune)."""
        _check(load().lutgemm_matvec_many_autotune(self._ws, self._xs, self._ys, self._ms, self.count, stream or None))

    def fused_plan(self):
        """Launch shape of the list's first launch: dict(entries, waves, k_blocks, measured)."""
        v = [ctypes.c_int() for _ in range(4)]
        _check(load().lutgemm_matvec_many_plan(self._ws, self._xs, self._ys, self._ms, self.count, *[ctypes.byref(x) for x in v]))
        return dict(entries=v[0].value, waves=v[1].value, k_blocks=v[2].value, measured=bool(v[3].value))


def read_probe(weights, stream=0):
    """Pure read of the packed tiles of each weight in turn (measurement aid), one C call."""
    arr = (ctypes.c_void_p * len(weights))(*[w._h for w in weights])
    _check(load().lutgemm_read_probe(arr, len(weights), stream or None))


def dense_gemv(wt_ptr, x_ptr, y_ptr, k, n, stream=0):
    """Comparator: y[n] = sum_k W^T[n][k] x[k] for a dense fp16 weight on the device (device
    pointers as integers)."""
    _check(load().lutgemm_dense_gemv_f16(wt_ptr, x_ptr, y_ptr, k, n, stream or None))


def version():
    return load().lutgemm_version().decode()
