"""Packed-weight files and the offline packer: host-side tests (no GPU) and, marked gpu, the
device round trip through lutgemm_weight_save / _load / _clone."""
import os
import struct
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLI = os.path.join(ROOT, "lut-gemm_amd", "lutgemm_pack")

SHAPES = [(1024, 100, 3, 64, True), (512, 32, 1, 512, False), (2048, 257, 4, 32, True), (96, 5, 8, 96, False)]


def problem(synth, k, n, q, g, offset, seed=0):
    return synth.make_weight(k, n, q, g, offset=offset, seed=seed)


@pytest.mark.parametrize("k,n,q,g,offset", SHAPES)
def test_pack_file_round_trip(lutgemm, tmp_path, k, n, q, g, offset):
    from lutgemm import synth
    w = problem(synth, k, n, q, g, offset)
    path = tmp_path / "w.lutw"
    lutgemm.pack_file(path, w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    u = lutgemm.unpack_file(path)
    assert (u["k"], u["n"], u["q"], u["num_groups"]) == (k, n, q, k // g)
    assert np.array_equal(u["bW"], w["bW"])
    assert np.array_equal(u["alpha"].astype(np.float32), w["alpha"])
    if offset:
        assert np.array_equal(u["q_bias"].astype(np.float32), w["q_bias"])
    else:
        assert u["q_bias"] is None
    # the file is the 64-byte header followed by exactly the device tiles
    sb, cb = lutgemm.packed_sizes(k, n, q, k // g, offset)
    assert os.path.getsize(path) == 64 + sb + cb
    raw = open(path, "rb").read()
    assert raw[:8] == b"LUTGEMMW"
    version, layout, fk, fn, fq, fg, foff = struct.unpack_from("<7I", raw, 8)
    assert (version, fk, fn, fq, fg, foff) == (1, k, n, q, k // g, int(offset))
    assert layout == 64 | (8 << 8) | (32 << 16)
    signs, scales = lutgemm.pack_host(w["bW"], lutgemm.float_to_half_bits(w["alpha"]),
                                      lutgemm.float_to_half_bits(w["q_bias"]) if offset else None, k, n, q, k // g)
    assert raw[64:64 + sb] == signs.tobytes() and raw[64 + sb:] == scales.tobytes()


def test_bad_files_are_refused(lutgemm, tmp_path):
    from lutgemm import synth
    w = problem(synth, 512, 40, 2, 128, False)
    path = tmp_path / "w.lutw"
    lutgemm.pack_file(path, w["bW"], w["alpha"], 512, 40, 2, 4, None)
    raw = open(path, "rb").read()
    cases = {
        "missing": None,
        "magic": b"NOTAFILE" + raw[8:],
        "version": raw[:8] + struct.pack("<I", 99) + raw[12:],
        "layout": raw[:12] + struct.pack("<I", 32 | (8 << 8) | (32 << 16)) + raw[16:],
        "truncated": raw[:-10],
        "shape": raw[:16] + struct.pack("<I", 500) + raw[20:],
        "short": raw[:20],
    }
    for name, data in cases.items():
        p = tmp_path / (name + ".lutw")
        if data is not None:
            p.write_bytes(data)
        with pytest.raises(lutgemm.LutGemmError) as e:
            lutgemm.unpack_file(p)
        assert e.value.status == lutgemm.ERR_IO, name
    with pytest.raises(lutgemm.LutGemmError) as e:
        lutgemm.pack_file(tmp_path / "no" / "such" / "dir.lutw", w["bW"], w["alpha"], 512, 40, 2, 4, None)
    assert e.value.status == lutgemm.ERR_IO
    with pytest.raises(lutgemm.LutGemmError) as e:
        lutgemm.pack_file(tmp_path / "x.lutw", w["bW"], w["alpha"], 512, 40, 2, 3, None)  # 512 % 3 != 0
    assert e.value.status == lutgemm.ERR_BAD_SHAPE


def test_command_line_packer(lutgemm, tmp_path):
    """lutgemm_pack pack / info / unpack on raw little-endian arrays in the reference layout."""
    from lutgemm import synth
    assert os.path.exists(CLI), "lutgemm_pack has not been built (make -C lut-gemm_amd/csrc)"
    k, n, q, g = 1024, 70, 3, 128
    w = problem(synth, k, n, q, g, True, seed=5)
    w["bW"].tofile(tmp_path / "bw.u32")
    w["alpha"].astype(np.float32).tofile(tmp_path / "alpha.f32")
    w["q_bias"].astype(np.float32).tofile(tmp_path / "qb.f32")
    out = tmp_path / "w.lutw"
    r = subprocess.run([CLI, "pack", "--k", str(k), "--n", str(n), "--q", str(q), "--groups", str(k // g),
                        "--bw", str(tmp_path / "bw.u32"), "--alpha", str(tmp_path / "alpha.f32"),
                        "--qbias", str(tmp_path / "qb.f32"), "-o", str(out)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    # same bytes as the library call
    lutgemm.pack_file(tmp_path / "ref.lutw", w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    assert out.read_bytes() == (tmp_path / "ref.lutw").read_bytes()
    r = subprocess.run([CLI, "info", str(out)], capture_output=True, text=True)
    assert r.returncode == 0 and "k=1024 n=70 q=3 num_groups=8 group_size=128 offset=1" in r.stdout
    r = subprocess.run([CLI, "unpack", str(out), "--bw", str(tmp_path / "bw2.u32"), "--alpha", str(tmp_path / "a2.f16"),
                        "--qbias", str(tmp_path / "z2.f16")], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(tmp_path / "bw2.u32", np.uint32), w["bW"].ravel())
    assert np.array_equal(np.fromfile(tmp_path / "a2.f16", np.float16).astype(np.float32), w["alpha"].ravel())
    assert np.array_equal(np.fromfile(tmp_path / "z2.f16", np.float16).astype(np.float32), w["q_bias"].ravel())
    # wrong input size and a file that is not a packed weight are reported, not packed
    r = subprocess.run([CLI, "pack", "--k", str(k), "--n", str(n + 1), "--q", str(q), "--groups", str(k // g),
                        "--bw", str(tmp_path / "bw.u32"), "--alpha", str(tmp_path / "alpha.f32"), "-o",
                        str(tmp_path / "bad.lutw")], capture_output=True, text=True)
    assert r.returncode != 0 and "does not hold exactly" in r.stderr
    r = subprocess.run([CLI, "info", str(tmp_path / "bw.u32")], capture_output=True, text=True)
    assert r.returncode != 0 and "not a packed-weight file" in r.stderr


def test_file_entry_points_check_their_arguments(lutgemm, tmp_path):
    """No device needed: null pointers and unreadable files are reported before any device work; a
    good file on a machine without a GPU fails with the no-device status, not with a crash."""
    import ctypes
    import torch
    from lutgemm import synth
    L = lutgemm.load()
    h = ctypes.c_void_p()
    assert L.lutgemm_weight_load(None, ctypes.byref(h)) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_load(b"/nonexistent/x.lutw", None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_load(b"/nonexistent/x.lutw", ctypes.byref(h)) == lutgemm.ERR_IO
    assert b"cannot open" in L.lutgemm_last_error()
    assert L.lutgemm_weight_save(None, b"/tmp/x.lutw") == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_weight_clone(None, ctypes.byref(h)) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_pack_file(None, None, None, 512, 8, 1, 1, b"/tmp/x.lutw") == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_unpack_file(None, None, None, None, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_read_probe(None, 1, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_read_probe((ctypes.c_void_p * 1)(None), 1, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_read_probe((ctypes.c_void_p * 1)(None), 0, None) == lutgemm.OK
    buf = (ctypes.c_uint16 * 64)()
    assert L.lutgemm_dense_gemv_f16(None, buf, buf, 64, 1, None) == lutgemm.ERR_NULL_POINTER
    assert L.lutgemm_dense_gemv_f16(buf, buf, buf, 60, 1, None) == lutgemm.ERR_BAD_SHAPE
    assert L.lutgemm_dense_gemv_f16(buf, buf, buf, 64, 0, None) == lutgemm.ERR_BAD_SHAPE
    assert L.lutgemm_status_string(lutgemm.ERR_IO) == b"file input/output failed"
    assert h.value is None
    if not torch.cuda.is_available():
        w = problem(synth, 512, 40, 2, 128, False)
        path = tmp_path / "w.lutw"
        lutgemm.pack_file(path, w["bW"], w["alpha"], 512, 40, 2, 4, None)
        with pytest.raises(lutgemm.LutGemmError) as e:
            lutgemm.BCQWeight.load(path)
        assert e.value.status == lutgemm.ERR_NO_DEVICE


@pytest.mark.gpu
@pytest.mark.parametrize("k,n,q,g,offset", [(2048, 300, 3, 128, True), (1536, 100, 2, 32, False)])
def test_save_load_clone_on_device(lutgemm, oracle, device, tmp_path, k, n, q, g, offset):
    from gpu_util import assert_within_tolerance, run_matvec
    from lutgemm import synth
    print("case files", k, n, q, g, offset, flush=True)
    w = problem(synth, k, n, q, g, offset, seed=k)
    x = synth.make_x(3, k, seed=1)
    W = lutgemm.BCQWeight(w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    W.set_plan(5, 2)
    y = run_matvec(lutgemm, W, x, device)
    z = w["q_bias"].astype(np.float16) if offset else None
    assert_within_tolerance(y, oracle.matvec_f64(w["bW"], w["alpha"].astype(np.float16), z, x), "original")

    path = tmp_path / "w.lutw"
    W.save(path)
    host = tmp_path / "host.lutw"
    lutgemm.pack_file(host, w["bW"], w["alpha"], k, n, q, k // g, w["q_bias"])
    assert path.read_bytes() == host.read_bytes()  # device tiles == host packer's tiles

    L = lutgemm.BCQWeight.load(path)
    assert (L.kSize, L.mSize, L.nb, L.num_groups, L.has_offset) == (k, n, q, k // g, offset)
    L.set_plan(5, 2)
    assert np.array_equal(run_matvec(lutgemm, L, x, device).view(np.uint16), y.view(np.uint16))
    C = W.clone()
    assert C.plan() == W.plan()
    assert np.array_equal(run_matvec(lutgemm, C, x, device).view(np.uint16), y.view(np.uint16))
    W.close()  # the clone owns its own device memory
    assert np.array_equal(run_matvec(lutgemm, C, x, device).view(np.uint16), y.view(np.uint16))
    bW2, a2, z2 = C.unpack()
    assert np.array_equal(bW2, w["bW"])
    C.close()
    L.close()
