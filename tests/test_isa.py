"""What the compiler made of the batch kernel, checked on the generated gfx950 assembly of the
library's own translation unit (no GPU needed: hipcc cross-compiles; about a minute).  The hot
loop and the end of a workgroup depend on properties the source can only ask for: the
transposition done by the LDS, the matrix instructions present, the index and the scale
multiply-add in one instruction each, no packed fp32 forms, no register used while an LDS read
into it is still in flight (the loop issues its reads ahead through asm statements and waits
with counts of its own), and, at the end, all answers of the split-k atomics awaited before the
first output is stored (a wait behind a store also waits for the store's round trip, which cost a
launch 1.5 to 2 microseconds when the compiler once arranged the code that way)."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "lut-gemm_amd", "csrc")


SOURCES = [("batch.hip", "lut_batch_kernel", "10MatvecArgs"), ("batch_multi.hip", "lut_batch_multi_kernel", "15MultiMatvecArgs")]


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """gfx950 assembly of the two translation units of the batch kernel, compiled side by side."""
    out_dir = tmp_path_factory.mktemp("isa")
    jobs = {}
    for source, _, _ in SOURCES:
        out = os.path.join(str(out_dir), source + ".s")
        cmd = ["/opt/rocm/bin/hipcc", "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Xclang", "-target-feature",
               "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I", CSRC, "-S", "--cuda-device-only",
               "-o", out, os.path.join(CSRC, source)]
        jobs[source] = (subprocess.Popen(cmd, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL), out)
    texts = {}
    for source, (proc, out) in jobs.items():
        assert proc.wait() == 0, source
        texts[source] = open(out).read()
    return texts


def kernels_of(text, kernel, args):
    found = {}
    for m in re.finditer(r"^(_ZN\S*%s(\S*?)EEvNS_%sE):[^\n]*\n(.*?)s_endpgm" % (kernel, args), text, re.S | re.M):
        body = [ln.strip() for ln in m.group(3).splitlines() if ln.strip() and not ln.strip().startswith(";")]
        meta = text[text.index(".amdhsa_kernel " + m.group(1)):]
        found[m.group(2)] = (body, meta[:meta.index(".end_amdhsa_kernel")])
    return found


def vgprs_named(operand):
    """VGPR numbers an operand names: v12, v[8:11]"""
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", operand):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


def uses_of_registers_in_flight(body):
    """LDS operations of a wavefront complete in order, and s_waitcnt lgkmcnt(n) returns when at most
    n are outstanding.  Walks the instructions in program order with that queue (kept across labels
    and branches, which only makes the check stricter) and returns the instructions that read or
    write a VGPR while an LDS read into it is queued."""
    queue, bad = [], []
    scalar_loads = False   # scalar memory loads count on the same counter and return in any order
    for line in body:
        line = line.split(";")[0].strip()
        if not line or line.endswith(":") or line.startswith("."):
            continue
        op, _, rest = line.partition(" ")
        operands = [o.strip() for o in rest.split(",")]
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", rest)
            if m:
                n = int(m.group(1))
                if n > 0 and scalar_loads and any(queue):
                    bad.append(line + "   ; partial wait for LDS reads with a scalar load outstanding")
                if n == 0:
                    scalar_loads = False
                queue = queue[len(queue) - n:] if 0 < n < len(queue) else ([] if n == 0 else queue)
            continue
        if op.startswith(("s_load_", "s_buffer_load_")):
            scalar_loads = True
            continue
        pending = set().union(*queue) if queue else set()
        if op.startswith("ds_"):
            is_read = "read" in op or "load" in op
            dest = vgprs_named(operands[0]) if is_read else set()
            sources = set().union(*[vgprs_named(o) for o in (operands[1:] if is_read else operands)])
            if (sources | dest) & pending:
                bad.append(line)
            queue.append(dest)
        elif set().union(*[vgprs_named(o) for o in operands]) & pending:
            bad.append(line)
    return bad


def test_the_in_flight_check_sees_a_short_wait():
    good = ["ds_read_b128 v[0:3], v9", "ds_read_b128 v[4:7], v9 offset:16", "s_waitcnt lgkmcnt(1)", "v_mov_b32_e32 v8, v0",
            "s_waitcnt lgkmcnt(0)", "v_mov_b32_e32 v8, v4"]
    assert uses_of_registers_in_flight(good) == []
    assert uses_of_registers_in_flight([good[0], good[1], "s_waitcnt lgkmcnt(1)", "v_mov_b32_e32 v8, v5"]) == ["v_mov_b32_e32 v8, v5"]
    assert uses_of_registers_in_flight([good[0], "ds_write_b32 v9, v2"]) == ["ds_write_b32 v9, v2"]
    # a scalar load shares the counter and may return after the LDS reads: a partial wait proves nothing
    mixed = ["s_load_dwordx2 s[0:1], s[4:5], 0x0", good[0], good[1], "s_waitcnt lgkmcnt(1)", "v_mov_b32_e32 v8, v0"]
    assert len(uses_of_registers_in_flight(mixed)) == 1
    assert uses_of_registers_in_flight([mixed[0], "s_waitcnt lgkmcnt(0)"] + good) == []


# register spills (scratch memory per lane, bytes) the instantiations may carry: none for two planes
# without offset, the headline of the decoder-layer chain; the largest ones are the offset variants
# with four scale groups per 128 k
MAX_SCRATCH_BYTES = 128


@pytest.mark.parametrize("source,kernel,args", SOURCES)
def test_batch_kernel_assembly(assembly, source, kernel, args):
    kernels = kernels_of(assembly[source], kernel, args)
    # 4 plane counts x offset x 3 scale layouts x second staged row, and for 5 to 8 planes the one
    # instantiation of eight wavefronts that stages two rows
    assert len(kernels) == 48 + 24, sorted(kernels)
    for name, (body, meta) in sorted(kernels.items()):
        ops = [ln.split()[0] for ln in body]
        q, offset, gsub, width, two = [int(v) for v in re.match(r"ILi(\d)ELb(\d)ELi(\d)ELi(\d+)ELb(\d)E", name).groups()]
        vgprs = int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", meta).group(1))
        # 16 wavefronts per workgroup fit a compute unit; more than four planes run with eight
        assert vgprs <= (128 if q <= 4 else 256), (name, vgprs)
        assert (width, two) == (8, 1) if q > 4 else width == 16, name
        assert ops.count("ds_read_b64_tr_b8") == 4 * q, name            # the transposition is the LDS's
        groups_of_32 = gsub == 4     # four scale groups per 128 k: the scales are the matrix operand, the offset term per output half
        assert ops.count("v_smfmac_f32_16x16x64_f16") == 32 * q + (32 if groups_of_32 else 16) * offset, name
        assert ops.count("v_and_or_b32") >= 16 * q, name                  # the index of a step: one instruction per sign word and parity
        assert "v_cvt_f32_f16_e32" not in ops, name                       # scales applied without conversions
        assert ops.count("v_fma_mix_f32") >= (0 if groups_of_32 else 32 * q), name
        assert uses_of_registers_in_flight(body) == [], name
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
        scratch = int(re.search(r"\.amdhsa_private_segment_fixed_size (\d+)", meta).group(1))
        assert scratch <= MAX_SCRATCH_BYTES, (name, scratch)
    # the headline instantiation of the decoder-layer chain (two planes, no offset, one group per 128 k): no scratch memory
    body, meta = kernels["ILi2ELb0ELi1ELi16ELb0E"]
    assert re.search(r"\.amdhsa_private_segment_fixed_size 0\b", meta)
