"""What the compiler made of the batch kernel, checked on the generated gfx950 assembly of the
library's own translation unit (no GPU needed: hipcc cross-compiles; about a minute).  The hot
loop and the end of a workgroup depend on properties the source can only ask for: the
transposition done by the LDS, the matrix instructions present, no packed fp32 forms, and, at the
end, all answers of the split-k atomics awaited before the first output is stored (a wait behind a
store also waits for the store's round trip, which cost a launch 1.5 to 2 microseconds when the
compiler once arranged the code that way)."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "lut-gemm_amd", "csrc")


def kernels_of(tmp_path, source):
    out = os.path.join(str(tmp_path), "out.s")
    cmd = ["/opt/rocm/bin/hipcc", "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature",
           "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", CSRC, "-S", "--cuda-device-only",
           "-o", out, os.path.join(CSRC, source)]
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    text = open(out).read()
    found = {}
    for m in re.finditer(r"^(_ZN\S*lut_batch_kernel(\S*?)EEvNS_10MatvecArgsE):[^\n]*\n(.*?)s_endpgm", text, re.S | re.M):
        body = [ln.strip() for ln in m.group(3).splitlines() if ln.strip() and not ln.strip().startswith(";")]
        meta = text[text.index(".amdhsa_kernel " + m.group(1)):]
        found[m.group(2)] = (body, meta[:meta.index(".end_amdhsa_kernel")])
    return found


def test_batch_kernel_assembly(tmp_path):
    kernels = kernels_of(tmp_path, "batch.hip")
    assert len(kernels) == 48, sorted(kernels)   # 4 plane counts x offset x 3 scale layouts x second staged row
    for name, (body, meta) in sorted(kernels.items()):
        ops = [ln.split()[0] for ln in body]
        q = int(re.match(r"ILi(\d)E", name).group(1))
        vgprs = int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", meta).group(1))
        assert vgprs <= 128, (name, vgprs)     # 16 wavefronts per workgroup fit a compute unit
        assert ops.count("ds_read_b64_tr_b8") == 4 * q, name            # the transposition is the LDS's
        offset = 1 if "ELb1ELi" in name[:12] else 0
        assert ops.count("v_mfma_f32_16x16x32_f16") == 32 * q + 16 * offset, name
        assert not any(op.startswith(("v_pk_add_f32", "v_pk_mul_f32", "v_pk_fma_f32")) for op in ops), name
        # the end: eight returning atomics, then one wait for all answers, then stores without waits between them
        atomics = [i for i, ln in enumerate(body) if ln.startswith("global_atomic_add_x2") and " sc0" in ln]
        assert len(atomics) == 8, (name, len(atomics))
        tail = body[atomics[-1] + 1:]
        stores = [i for i, ln in enumerate(tail) if ln.startswith("global_store_short")]
        assert len(stores) >= 8, name
        waits_before = [ln for ln in tail[:stores[0]] if ln.startswith("s_waitcnt") and "vmcnt" in ln]
        assert waits_before and "vmcnt(0)" in waits_before[-1], (name, waits_before)
        between = tail[stores[0]:stores[7]]   # (the stores of the path without k-splits follow behind a branch of their own)
        assert not [ln for ln in between if ln.startswith("s_waitcnt") and "vmcnt" in ln], name
    # the headline instantiation of the decoder-layer chain (two planes, no offset, one group per 128 k): no scratch memory
    body, meta = kernels["ILi2ELb0ELi1ELi16ELb0E"]
    assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", meta)
