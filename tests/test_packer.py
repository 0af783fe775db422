"""Host logic of the product that needs no GPU: the wave64 re-tiling (bijection, documented
index formula), the ingest rounding, argument validation of the C ABI, and that the shared
library exports every symbol the header declares."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def problem(rng, K, N, q, g, offset):
    bW = rng.integers(0, 2 ** 32, size=(K // 32, q, N), dtype=np.uint32)
    alpha = rng.normal(0, 1, size=(K // g, q, N)).astype(np.float16).view(np.uint16)
    z = rng.normal(0, 1, size=(K // g, N)).astype(np.float16).view(np.uint16) if offset else None
    return bW, alpha, z


SHAPES = [  # K, N, q, g, offset  (ragged n, ragged k-blocks, all three scale-group modes)
    (512, 32, 3, 128, False), (512, 32, 3, 128, True), (1024, 64, 1, 64, False), (1536, 96, 2, 32, True),
    (32, 1, 1, 32, False), (96, 33, 4, 96, True), (640, 70, 8, 128, False), (2048, 40, 3, 2048, True),
    (1024, 17, 5, 256, False), (192, 100, 2, 64, True), (4096, 8, 3, 128, False),
]


@pytest.mark.parametrize("K,N,q,g,offset", SHAPES)
def test_pack_unpack_round_trip(lutgemm, K, N, q, g, offset):
    rng = np.random.default_rng(K + N + q)
    bW, alpha, z = problem(rng, K, N, q, g, offset)
    signs, scales = lutgemm.pack_host(bW, alpha, z, K, N, q, K // g)
    sb, cb = lutgemm.packed_sizes(K, N, q, K // g, offset)
    assert signs.nbytes == sb and scales.nbytes == cb
    bW2, alpha2, z2 = lutgemm.unpack_host(signs, scales, K, N, q, K // g, offset)
    assert np.array_equal(bW2, bW)
    assert np.array_equal(alpha2, alpha)
    if offset:
        assert np.array_equal(z2, z)


@pytest.mark.parametrize("K,N,q,g,offset", [(1024, 64, 3, 128, True), (1024, 40, 2, 64, False), (512, 64, 2, 32, True)])
def test_tile_index_formula(lutgemm, K, N, q, g, offset):
    """Every byte / half of the tiles sits where the documented layout says (brute force)."""
    rng = np.random.default_rng(42)
    bW, alpha, z = problem(rng, K, N, q, g, offset)
    signs, scales = lutgemm.pack_host(bW, alpha, z, K, N, q, K // g)
    TS, NB = (K + 511) // 512, (N + 31) // 32
    qo = q + int(offset)
    gsub = 1 if g % 128 == 0 else 2 if g % 64 == 0 else 4
    subl, lh = 16 // gsub, 2 * gsub * qo
    signs = signs.reshape(NB, TS, 2 * q, 64, 16)
    scales = scales.reshape(NB, TS, 64, 2 * gsub, qo)
    for _ in range(3000):
        nb, ts, b, h, lane, p = (rng.integers(0, m) for m in (NB, TS, q, 2, 64, 16))
        c, n = ts * 64 + lane, nb * 32 + h * 16 + p
        want = 0
        if c < K // 8 and n < N:
            want = (int(bW[c // 4, b, n]) >> (8 * (c % 4))) & 0xFF
        assert signs[nb, ts, 2 * b + h, lane, p] == want
    for _ in range(3000):
        nb, ts, lane, t, bo = (rng.integers(0, m) for m in (NB, TS, 64, 2 * gsub, qo))
        r, j = lane // 16, lane % 16
        kpos = ts * 512 + r * 128 + (j // subl) * (128 // gsub)
        n = nb * 32 + t * subl + (j % subl)
        want = 0
        if kpos < K and n < N:
            want = alpha[kpos // g, bo, n] if bo < q else z[kpos // g, n]
        assert scales[nb, ts, lane, t, bo] == want
    assert lh == scales.shape[3] * scales.shape[4]


def test_ingest_rounding_is_rne(lutgemm):
    rng = np.random.default_rng(0)
    v = np.concatenate([rng.normal(0, 1, 100000), rng.normal(0, 1e-6, 20000), rng.normal(0, 4e4, 20000),
                        [0.0, -0.0, 65504.0, 65520.0, 2.0 ** -25, 1.5 * 2.0 ** -25, 2.0 ** -24]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = v.astype(np.float16).view(np.uint16)
    assert np.array_equal(lutgemm.float_to_half_bits(v), want)


def test_header_symbols_are_exported(lutgemm):
    """Every function declared in include/lutgemm_c.h resolves in the shared library."""
    text = open(os.path.join(ROOT, "include", "lutgemm_c.h")).read()
    declared = set(re.findall(r"\b(lutgemm_[a-z0-9_]+)\s*\(", text))
    declared -= {"lutgemm_status"}
    assert declared == set(lutgemm.EXPORTED)
    L = lutgemm.load()
    for name in sorted(declared):
        assert getattr(L, name) is not None
    assert lutgemm.version().startswith("lutgemm-hip")


def test_argument_validation_without_device(lutgemm):
    L = lutgemm.load()
    h = ctypes.c_void_p()
    bW = np.zeros((4, 1, 8), np.uint32)
    a = np.zeros((1, 1, 8), np.float32)
    P = lambda x: x.ctypes.data_as(ctypes.c_void_p)
    cases = [  # k, n, q, num_groups
        (100, 8, 1, 1),   # k not a multiple of 32
        (128, 0, 1, 1),   # n == 0
        (128, 8, 0, 1),   # q == 0
        (128, 8, 9, 1),   # q > 8
        (128, 8, 1, 3),   # k % num_groups != 0
        (128, 8, 1, 8),   # group length 16 is not a multiple of 32
        (128, 8, 1, 0),
    ]
    for k, n, q, G in cases:
        st = L.lutgemm_weight_create(P(bW), P(a), None, k, n, q, G, ctypes.byref(h))
        assert st == lutgemm.ERR_BAD_SHAPE, (k, n, q, G)
        assert h.value is None
        assert b"bad shape" in L.lutgemm_last_error()
    assert L.lutgemm_weight_create(None, P(a), None, 128, 8, 1, 1, ctypes.byref(h)) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_create(P(bW), None, None, 128, 8, 1, 1, ctypes.byref(h)) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_create(P(bW), P(a), None, 128, 8, 1, 1, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_matvec(None, None, None, 1, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_destroy(None) == lutgemm.OK          # destroying nothing is fine
    assert L.lutgemm_weight_info(None, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_status_string(2) == b"bad shape"
    with pytest.raises(lutgemm.LutGemmError):
        lutgemm.packed_sizes(100, 8, 1, 1, False)
    with pytest.raises(lutgemm.LutGemmError):                    # python mirror checks array sizes
        lutgemm.BCQWeight(bW, a, 256, 8, 1, 1)


def test_create_without_gpu_fails_loudly(lutgemm):
    """On a machine without a HIP device the product refuses to run: no CPU fallback."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; this checks the no-device error path")
    bW = np.zeros((4, 1, 8), np.uint32)
    a = np.zeros((1, 1, 8), np.float32)
    with pytest.raises(lutgemm.LutGemmError) as e:
        lutgemm.BCQWeight(bW, a, 128, 8, 1, 1)
    assert e.value.status == lutgemm.ERR_NO_DEVICE
