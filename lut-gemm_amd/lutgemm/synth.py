"""Seeded synthetic BCQ problems: the benchmark configurations and arbitrary small shapes.

Distributions follow the benchmark definition: sign planes Bernoulli(0.5) packed 32 per uint32
in the reference's [k/32][q][n] layout, scales |N(0, 0.02)| (0.02 and 0.01 are standard
deviations), activations N(0, 1) rounded to fp16.  The "rtn" variant is uniform 4-bit codes
written as BCQ with an offset (alpha_i = s * 2^i / 2, offset ~ N(0, 0.01)), the closed form of
examples/rtn_parameter.py:77-96 with the offset drawn directly.
All draws come from numpy's PCG64 with an explicit seed, so both machines see the same data.
"""
import zlib

import numpy as np

CONFIGS = {
    # name: m, k, n, q, g, offset/rtn
    "cfg0": dict(m=1, k=4096, n=4096, q=3, g=128, rtn=False),
    "cfg1": dict(m=1, k=12288, n=12288, q=3, g=128, rtn=False),
    "cfg2": dict(m=1, k=12288, n=49152, q=4, g=128, rtn=True),
}
# cfg3: k=n=7168, q in 1..4, g in {32, 64, 128, k}
CFG3_POINTS = [dict(m=1, k=7168, n=7168, q=q, g=g, rtn=False) for q in (1, 2, 3, 4) for g in (32, 64, 128, 7168)]
# cfg4: q=2, g=128, m in {1,2,4,8}, four decoder-layer shapes
CFG4_LAYERS = {
    "qkv": dict(k=12288, n=36864), "out": dict(k=12288, n=12288),
    "fc1": dict(k=12288, n=49152), "fc2": dict(k=49152, n=12288),
}


def _rng(seed, tag):
    return np.random.Generator(np.random.PCG64([seed, zlib.crc32(tag.encode())]))


def make_weight(k, n, q, g, rtn=False, offset=None, seed=0):
    """Returns dict(bW uint32 [k/32][q][n], alpha float32 [G][q][n], q_bias float32 [G][n] | None).

    offset=None means "offset iff rtn".  alpha / q_bias values are exactly representable in fp16.
    """
    G = k // g
    has_off = rtn if offset is None else offset
    bW = _rng(seed, "signs").integers(0, 2 ** 32, size=(k // 32, q, n), dtype=np.uint32)
    if rtn:
        s = np.abs(_rng(seed, "scale").normal(0.0, 0.02, size=(G, n))).astype(np.float16).astype(np.float32)
        alpha = np.stack([s * (2.0 ** b) / 2.0 for b in range(q)], axis=1)
    else:
        alpha = np.abs(_rng(seed, "alpha").normal(0.0, 0.02, size=(G, q, n)))
    alpha = alpha.astype(np.float16).astype(np.float32)
    q_bias = None
    if has_off:
        q_bias = _rng(seed, "offset").normal(0.0, 0.01, size=(G, n)).astype(np.float16).astype(np.float32)
    return dict(bW=bW, alpha=alpha, q_bias=q_bias, k=k, n=n, q=q, g=g, num_groups=G)


def make_x(m, k, seed=0):
    return _rng(seed, "x").normal(0.0, 1.0, size=(m, k)).astype(np.float16)


def algorithmic_bytes(k, n, q, g, has_offset, m=1):
    """(B_w packed-weight bytes, B total bytes) of one matvec."""
    b_sign = k * n * q // 8
    b_alpha = (k // g) * q * n * 2
    b_off = (k // g) * n * 2 if has_offset else 0
    b_w = b_sign + b_alpha + b_off
    return b_w, b_w + m * k * 2 + m * n * 2
