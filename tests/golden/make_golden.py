"""Writes the small known-answer fixtures of tests/golden/*.npz.

The reference holds no data files or known-answer vectors for this path, and none of its code is
imported or run here: inputs come from the seeded generator of this repository and the expected
outputs from the CPU oracle (double-precision truth) after the oracle itself has been pinned by
tests/test_oracle.py.  The fixtures freeze those answers so that a later change to the oracle, the
generator or the library shows up as a diff against committed data.  Beside every .npz lies the
packed-weight file (.lutw) the host packer writes for it: a change of the tile layout or of the
file format shows up the same way.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "lut-gemm_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

CASES = [  # name, k, n, q, g, offset, rtn, m
    ("k64_n8_q1_g32", 64, 8, 1, 32, False, False, 1),
    ("k64_n8_q3_g64_off", 64, 8, 3, 64, True, False, 1),
    ("k512_n40_q3_g128", 512, 40, 3, 128, False, False, 2),
    ("k1024_n33_q4_g128_rtn", 1024, 33, 4, 128, True, True, 1),
    ("k1536_n64_q2_g32_off", 1536, 64, 2, 32, True, False, 3),
]


def main():
    from lutgemm import synth
    from oracle import oracle
    for name, k, n, q, g, off, rtn, m in CASES:
        w = synth.make_weight(k, n, q, g, rtn=rtn, offset=off, seed=7)
        x = synth.make_x(m, k, seed=7)
        z = w["q_bias"].astype(np.float16) if w["q_bias"] is not None else None
        y = oracle.matvec_f64(w["bW"], w["alpha"].astype(np.float16), z, x)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), bW=w["bW"], alpha=w["alpha"].astype(np.float16),
                            q_bias=(z if z is not None else np.zeros(0, np.float16)), x=x, y=y,
                            meta=np.array([k, n, q, g, int(off), m]))
        # the packed-weight file of the same problem: freezes the tile layout and the file format
        import lutgemm
        lutgemm.pack_file(os.path.join(HERE, name + ".lutw"), w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
        print(name, y.shape, float(np.abs(y).max()))


if __name__ == "__main__":
    main()
