"""Committed known-answer fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must still give the stored answers (CPU), and the HIP library must match them (GPU)."""
import glob
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FILES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def load(path):
    d = np.load(path)
    k, n, q, g, off, m = (int(v) for v in d["meta"])
    z = d["q_bias"] if off else None
    return d["bW"], d["alpha"], z, d["x"], d["y"], (k, n, q, g, m)


def test_fixtures_exist():
    assert len(FILES) >= 5


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_oracle_reproduces_fixture(oracle, path):
    bW, alpha, z, x, y, _ = load(path)
    got = oracle.matvec_f64(bW, alpha, z, x)
    assert np.allclose(got, y, rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_packed_file_fixture_is_reproduced(lutgemm, tmp_path, path):
    """The committed packed-weight file of each fixture: today's host packer writes the same
    bytes (tile layout and file format unchanged) and reads the stored arrays back from it."""
    bW, alpha, z, _, _, (k, n, q, g, _) = load(path)
    stored = path[:-4] + ".lutw"
    fresh = tmp_path / "fresh.lutw"
    lutgemm.pack_file(fresh, bW, alpha, k, n, q, k // g, z)
    assert fresh.read_bytes() == open(stored, "rb").read()
    u = lutgemm.unpack_file(stored)
    assert (u["k"], u["n"], u["q"], u["num_groups"]) == (k, n, q, k // g)
    assert np.array_equal(u["bW"], bW) and np.array_equal(u["alpha"], alpha)
    assert (u["q_bias"] is None) == (z is None) and (z is None or np.array_equal(u["q_bias"], z))


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_library_loads_packed_file_fixture(lutgemm, device, path):
    from gpu_util import assert_within_tolerance, run_matvec
    _, _, _, x, y, _ = load(path)
    W = lutgemm.BCQWeight.load(path[:-4] + ".lutw")
    assert_within_tolerance(run_matvec(lutgemm, W, x, device), y, os.path.basename(path) + " from file")
    W.close()


@pytest.mark.gpu
@pytest.mark.parametrize("path", FILES, ids=[os.path.basename(f)[:-4] for f in FILES])
def test_library_matches_fixture(lutgemm, device, path):
    from gpu_util import assert_within_tolerance, run_matvec
    bW, alpha, z, x, y, (k, n, q, g, m) = load(path)
    print("case golden", os.path.basename(path), flush=True)
    W = lutgemm.BCQWeight(bW, alpha, k, n, q, k // g, z)
    assert_within_tolerance(run_matvec(lutgemm, W, x, device), y, os.path.basename(path))
    W.close()
