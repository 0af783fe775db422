"""Pins the CPU oracle (oracle/lutgemm_oracle.c) against things it does not compute itself:
numpy.float16 conversions, numpy bit unpacking + dense float64 matmul, closed forms and
brute force on tiny inputs.  The reference holds no golden vectors for this path
(its only test prints latencies), so these are what fixes the oracle.
"""
import numpy as np
import pytest


def unpack_signs_np(bW, K):
    """Independent unpacking: +1/-1 [K][q][N] from bW [K/32][q][N] via numpy bit ops."""
    KW, q, N = bW.shape
    bits = ((bW[:, None, :, :] >> np.arange(32, dtype=np.uint32)[None, :, None, None]) & 1)
    return (bits.reshape(K, q, N).astype(np.int8) * 2 - 1)


def dense_np(bW, alpha16, zoff16, K, g):
    """Textbook dense W[k][n] in float64 from the container definition."""
    s = unpack_signs_np(bW, K).astype(np.float64)               # [K][q][N]
    a = np.repeat(alpha16.astype(np.float64), g, axis=0)          # [K][q][N]
    W = (s * a).sum(axis=1)
    if zoff16 is not None:
        W = W + np.repeat(zoff16.astype(np.float64), g, axis=0)
    return W


def rand_problem(rng, K, N, q, g, offset):
    bW = rng.integers(0, 2 ** 32, size=(K // 32, q, N), dtype=np.uint32)
    alpha = np.abs(rng.normal(0, 0.02, size=(K // g, q, N))).astype(np.float16)
    z = rng.normal(0, 0.01, size=(K // g, N)).astype(np.float16) if offset else None
    x = rng.normal(0, 1, size=(1, K)).astype(np.float16)
    return bW, alpha, z, x


# ---------------------------------------------------------------- fp16 conversion
def test_f2h_matches_numpy_on_all_halves_and_neighbours(oracle):
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(f)
    assert np.array_equal(oracle.h2f(h)[finite], f[finite])
    assert np.array_equal(oracle.f2h(f)[finite], h[finite])
    # values between representable halves, ties included: nudge by fractions of the spacing
    base = f[finite & (h < 0x7c00)]
    with np.errstate(over="ignore"):
        nxt = np.nextafter(base.astype(np.float16), np.float16(np.inf)).astype(np.float32)
    for frac in (0.25, 0.5, 0.75):
        v = (base + (nxt - base) * np.float32(frac)).astype(np.float32)
        v = v[np.isfinite(v)]
        assert np.array_equal(oracle.f2h(v), v.astype(np.float16).view(np.uint16))
        assert np.array_equal(oracle.f2h(-v), (-v).astype(np.float16).view(np.uint16))


def test_f2h_and_d2h_random_and_specials(oracle):
    rng = np.random.default_rng(1)
    v = np.concatenate([
        rng.normal(0, 1, 200000), rng.normal(0, 1e-5, 50000), rng.normal(0, 3e4, 50000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  1.5 * 2.0 ** -25, 2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, np.inf, -np.inf]),
    ])
    with np.errstate(over="ignore"):
        want32 = v.astype(np.float32).astype(np.float16).view(np.uint16)
        want64 = v.astype(np.float64).astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f2h(v.astype(np.float32)), want32)
    assert np.array_equal(oracle.d2h(v), want64)


# ---------------------------------------------------------------- packing convention
def test_pack_signs_bit_convention(oracle):
    rng = np.random.default_rng(2)
    K, q, N = 96, 3, 5
    signs = rng.choice(np.array([-1, 1], np.int8), size=(K, q, N))
    bW = oracle.pack_signs(signs)
    # brute force: bit t of word w is weight 32 w + t, set means +1
    for k in range(K):
        for b in range(q):
            for n in range(N):
                bit = (int(bW[k // 32, b, n]) >> (k % 32)) & 1
                assert bit == (1 if signs[k, b, n] > 0 else 0)
    assert np.array_equal(unpack_signs_np(bW, K), signs)


# ---------------------------------------------------------------- dequantize_cpu
@pytest.mark.parametrize("K,N,q,g", [(64, 8, 1, 32), (128, 7, 3, 64), (256, 16, 4, 128), (128, 5, 2, 128)])
def test_dequantize_cpu_bit_exact_vs_numpy(oracle, K, N, q, g):
    rng = np.random.default_rng(3)
    bW, alpha, _, _ = rand_problem(rng, K, N, q, g, False)
    got = oracle.dequantize_cpu(bW, alpha)
    # same arithmetic in numpy: float32 running sum over planes in ascending order, one rounding
    s = unpack_signs_np(bW, K).astype(np.float32)
    a = np.repeat(alpha.astype(np.float32), g, axis=0)
    acc = np.zeros((K, N), np.float32)
    for b in range(q):
        acc = acc + s[:, b, :] * a[:, b, :]
    assert np.array_equal(got.view(np.uint16), acc.astype(np.float16).view(np.uint16))
    # row-wise orientation is the transpose
    assert np.array_equal(oracle.dequantize_cpu(bW, alpha, row_wise=True), got.T)
    # and it ignores any offset by construction: equals the offset-free dense weight
    assert np.allclose(got.astype(np.float64), dense_np(bW, alpha, None, K, g), atol=2e-3 * 0.1)


def test_dequantize_omp_equals_serial(oracle):
    rng = np.random.default_rng(4)
    bW, alpha, _, _ = rand_problem(rng, 256, 33, 3, 128, False)
    a = oracle.dequantize_cpu(bW, alpha)
    b, used = oracle.dequantize_cpu_omp(bW, alpha)
    assert used >= 1 and np.array_equal(a.view(np.uint16), b.view(np.uint16))


# ---------------------------------------------------------------- matmul_cpu
def test_matmul_cpu_exact_on_integers_and_close_on_random(oracle):
    rng = np.random.default_rng(5)
    x = rng.integers(-8, 9, size=(3, 64)).astype(np.float16)
    W = rng.integers(-8, 9, size=(64, 10)).astype(np.float16)
    want = x.astype(np.int64) @ W.astype(np.int64)
    assert np.array_equal(oracle.matmul_cpu(x, W).astype(np.int64), want)
    x = rng.normal(0, 1, size=(2, 512)).astype(np.float16)
    W = rng.normal(0, 0.05, size=(512, 9)).astype(np.float16)
    ref = x.astype(np.float64) @ W.astype(np.float64)
    got = oracle.matmul_cpu(x, W)
    assert np.allclose(got, ref, rtol=0, atol=512 * 2.0 ** -24 * 4)
    par, used = oracle.matmul_cpu_omp(x, W)
    assert used >= 1 and np.array_equal(par, got)


# ---------------------------------------------------------------- the double-precision truth
@pytest.mark.parametrize("K,N,q,g,offset", [
    (64, 8, 1, 32, False), (128, 9, 3, 64, True), (512, 33, 3, 128, False),
    (1024, 40, 4, 128, True), (256, 6, 2, 256, True), (96, 3, 5, 32, False)])
def test_matvec_f64_vs_dense_numpy(oracle, K, N, q, g, offset):
    rng = np.random.default_rng(6)
    bW, alpha, z, _ = rand_problem(rng, K, N, q, g, offset)
    x = rng.normal(0, 1, size=(3, K)).astype(np.float16)
    W = dense_np(bW, alpha, z, K, g)
    want = x.astype(np.float64) @ W
    got = oracle.matvec_f64(bW, alpha, z, x)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert np.allclose(oracle.dense_weight_f64(bW, alpha, z), W, rtol=0, atol=1e-15)


def test_matvec_f64_special_cases(oracle):
    rng = np.random.default_rng(7)
    K, N, g = 256, 12, 128
    x = rng.normal(0, 1, size=(1, K)).astype(np.float16)
    sx = x.astype(np.float64).sum()
    ones = np.ones((K // g, 1, N), np.float16)
    all1 = np.full((K // 32, 1, N), 0xFFFFFFFF, np.uint32)
    all0 = np.zeros((K // 32, 1, N), np.uint32)
    assert np.allclose(oracle.matvec_f64(all1, ones, None, x), sx, atol=1e-12)      # every sign +1
    assert np.allclose(oracle.matvec_f64(all0, ones, None, x), -sx, atol=1e-12)     # every sign -1
    # single-hot activation picks one row of W
    bW, alpha, z, _ = rand_problem(rng, K, N, 3, g, True)
    W = dense_np(bW, alpha, z, K, g)
    for k in (0, 31, 32, 127, 128, 255):
        e = np.zeros((1, K), np.float16)
        e[0, k] = 1
        assert np.allclose(oracle.matvec_f64(bW, alpha, z, e)[0], W[k], atol=1e-15)
    # additivity over bit planes and linearity in alpha
    y = oracle.matvec_f64(bW, alpha, None, x)
    parts = sum(oracle.matvec_f64(bW[:, b:b + 1], alpha[:, b:b + 1], None, x) for b in range(3))
    assert np.allclose(y, parts, atol=1e-12)
    assert np.allclose(oracle.matvec_f64(bW, (alpha * np.float16(2)).astype(np.float16), None, x), 2 * y, atol=1e-12)
    # offset identity: y_with - y_without = sum_g z[g][n] * sum_{k in g} x[k]
    yz = oracle.matvec_f64(bW, alpha, z, x)
    xs = x.astype(np.float64).reshape(K // g, g).sum(axis=1)
    assert np.allclose(yz - y, xs @ z.astype(np.float64), atol=1e-12)
    # one group over all k equals two groups with duplicated scales
    a1 = alpha[:1]
    a2 = np.concatenate([a1, a1], axis=0)
    assert np.allclose(oracle.matvec_f64(bW, a1, None, x), oracle.matvec_f64(bW, a2, None, x), atol=1e-12)


def test_matvec_f64_integer_code_reduces_to_integer_gemv(oracle):
    """alpha_b = 2^b / 2 with the bits of an integer code c gives W = c - (2^q - 1)/2."""
    rng = np.random.default_rng(8)
    K, N, q = 128, 10, 4
    codes = rng.integers(0, 16, size=(K, N)).astype(np.uint8)
    bW, alpha, off = oracle.rtn_to_bcq(codes, np.ones((1, N), np.float32), np.zeros((1, N), np.float32), q, K)
    x = rng.integers(-4, 5, size=(1, K)).astype(np.float16)
    want = x.astype(np.int64) @ codes.astype(np.int64)           # integer GEMV of the raw codes
    got = oracle.matvec_f64(bW, alpha.astype(np.float16), off.astype(np.float16), x)
    assert np.array_equal(np.rint(got).astype(np.int64), want) and np.allclose(got, want, atol=1e-9)


# ---------------------------------------------------------------- LUT closed form
def test_lut256_closed_form_and_symmetries(oracle):
    rng = np.random.default_rng(9)
    x8 = rng.normal(0, 1, 8).astype(np.float16)
    lut = oracle.lut256_f64(x8)
    xf = x8.astype(np.float64)
    for idx in range(256):
        want = sum(xf[j] if (idx >> j) & 1 else -xf[j] for j in range(8))
        assert abs(lut[idx] - want) < 1e-14
    assert np.allclose(lut[::-1], -lut, atol=1e-15)               # lut[255 - i] = -lut[i]
    assert abs(lut[255] - xf.sum()) < 1e-14 and abs(lut[0] + xf.sum()) < 1e-14


# ---------------------------------------------------------------- RTN -> BCQ closed form
def test_rtn_to_bcq_identity_exhaustive(oracle):
    q, g, K = 4, 32, 32
    codes = np.arange(16, dtype=np.uint8).reshape(1, 16).repeat(K, axis=0)      # column n has code n
    scale = np.full((1, 16), 0.0371, np.float32)
    zero = np.full((1, 16), 7.0, np.float32)
    bW, alpha, off = oracle.rtn_to_bcq(codes, scale, zero, q, g)
    bits = unpack_signs_np(bW, K).astype(np.float64)
    w = (bits * alpha.astype(np.float64)[0][None]).sum(axis=1) + off.astype(np.float64)[0][None]
    want = scale.astype(np.float64) * (codes.astype(np.float64) - zero.astype(np.float64))
    assert np.allclose(w, want, atol=1e-7)
    assert np.allclose(alpha[0, :, 0], scale[0, 0] * np.array([0.5, 1, 2, 4]), rtol=1e-6)   # ascending, LSB first


# ---------------------------------------------------------------- fp16 emulation of the reference kernels
@pytest.mark.parametrize("offset", [False, True])
def test_ref_kernel_emulation_exact_when_nothing_rounds(oracle, offset):
    """With small integer activations and unit scales every fp16 operation is exact, so the
    emulated kernel must reproduce the truth exactly.  (The order of its rounding steps is pinned
    in test_oracle_ref_kernel.py.)"""
    rng = np.random.default_rng(10)
    K, N, q, g = 256, 8, 3, 128
    bW = rng.integers(0, 2 ** 32, size=(K // 32, q, N), dtype=np.uint32)
    alpha = np.ones((K // g, q, N), np.float16)
    z = np.full((K // g, N), 2.0, np.float16) if offset else None
    x = rng.integers(-2, 3, size=(1, K)).astype(np.float16)
    truth = oracle.matvec_f64(bW, alpha, z, x)[0]
    for fused in (False, True):
        y = oracle.ref_kernel_fp16(bW, alpha, z, x, fused=fused).astype(np.float64)
        assert np.array_equal(y, truth)


def test_ref_kernel_emulation_close_on_random(oracle):
    rng = np.random.default_rng(11)
    K, N, q, g = 1024, 64, 3, 128
    bW, alpha, z, x = rand_problem(rng, K, N, q, g, True)
    for zz in (None, z):
        truth = oracle.matvec_f64(bW, alpha, zz, x)[0]
        y = oracle.ref_kernel_fp16(bW, alpha, zz, x[0])
        mean_abs, max_abs, rel = oracle.error_stats(y, truth)
        assert max_abs < 0.05 and rel < 2e-2           # fp16 accumulation error, loose sanity bound
        assert max_abs > 0                             # it does round: it is not the truth in disguise


def test_error_stats(oracle):
    y = np.array([1.0, 2.0, 4.0], np.float16)
    t = np.array([1.5, 2.0, 3.0], np.float64)
    mean_abs, max_abs, rel = oracle.error_stats(y, t)
    assert abs(mean_abs - 0.5) < 1e-12 and abs(max_abs - 1.0) < 1e-12
    assert abs(rel - np.sqrt(1.25 / 15.25)) < 1e-12
