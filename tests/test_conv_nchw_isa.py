"""The staging registers of the NCDHW-direct convolution's loader waves belong to their assembly
statements alone (amos_amd/isa_check.py says why that matters and what is checked; the build runs
the same check before it links).  This test compiles every instance to assembly -- no GPU needed --
and reads it, and checks the checker on doctored code."""
import os
import subprocess
import tempfile

import pytest

from amos_amd import build as amos_build
from amos_amd import isa_check


def _compile_all(tmp):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    procs = []
    for u in isa_check.UNITS:
        out = os.path.join(tmp, u + ".s")
        log = open(os.path.join(tmp, u + ".log"), "w+")
        cmd = [hipcc] + amos_build.HIP_FLAGS + ["-I" + os.path.join(amos_build.ROOT, "include"), "-I" + amos_build.CSRC] + \
            isa_check.ASM_FLAGS + [os.path.join(amos_build.CSRC, u), "-o", out]
        procs.append((u, out, log, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT)))
    res = []
    for u, out, log, p in procs:
        rc = p.wait()
        log.seek(0)
        text = log.read()
        log.close()
        assert rc == 0, "hipcc failed on %s:\n%s" % (u, text[-3000:])
        res.append((u, out, text))
    return res


@pytest.mark.timeout(900)
def test_staging_registers_belong_to_the_assembly_statements():
    with tempfile.TemporaryDirectory() as tmp:
        total, bad = 0, []
        for unit, asm, log in _compile_all(tmp):
            n, b = isa_check.violations(unit, asm, log)
            total += n
            bad += b
        assert not bad, "\n".join(bad)
        assert total >= 100


def test_the_check_sees_a_violation(tmp_path):
    """doctored code: a compiler-generated instruction that names a staging register, an assembly
    statement outside the staging range, a spill -- each must be reported"""
    sym = "_ZN4amos14amos_conv_nchwILi0ELi64ELi128ELi2ELi4ELi1ELi2ELi4ELi8EEEvNS_14ConvNchwParamsE"
    # a staging load, compiler code behind it (HERE), the wait, code behind the wait (AFTER), and a
    # block that only the matrix-core waves run (a branch around the loaders' code: OTHER)
    good = ("%s:\n\ts_cbranch_scc1 .LBB0_2\n\tv_mov_b32_e32 v5, 0\n"
            "\t;;#ASMSTART\n\tglobal_load_dwordx2 v[136:137], v5, s[0:1]\n\t;;#ASMEND\n"
            "\tv_mov_b32_e32 v6, 1\n"                                      # HERE
            "\t;;#ASMSTART\n\ts_waitcnt vmcnt(0)\n\t;;#ASMEND\n"
            "\tv_mov_b32_e32 v7, 2\n\ts_endpgm\n"                         # AFTER
            ".LBB0_2:\n\tv_mov_b32_e32 v8, 3\n\ts_endpgm\n.Lfunc_end0:\n" % sym)   # OTHER
    log = "remark: Function Name: %s\nremark:     VGPRs: 168\nremark:     AGPRs: 0\nremark:     ScratchSize [bytes/lane]: 0\nremark:     Occupancy [waves/SIMD]: 3\n" % sym

    def run(asm, remarks=log):
        path = tmp_path / "x.s"
        path.write_text(asm)
        return isa_check.violations("x", str(path), remarks)[1]

    assert run(good) == []
    # between the load and its wait: reported, whether the register is written or read, alone or in a range
    assert any("names a staging register" in b for b in run(good.replace("v_mov_b32_e32 v6, 1", "v_add_u32_e32 v140, v5, v5")))
    assert any("names a staging register" in b for b in run(good.replace("v_mov_b32_e32 v6, 1", "ds_read_b128 v[134:137], v5")))
    # ... also where the stretch runs through a branch target
    assert any("names a staging register" in b
               for b in run(good.replace("v_mov_b32_e32 v6, 1", "s_cbranch_scc0 .LBB0_2").replace("v_mov_b32_e32 v8, 3", "v_mov_b32_e32 v150, 3")))
    # behind the wait, and in code that no path from a staging load reaches before a wait: the
    # data has landed / these are other waves' registers
    assert run(good.replace("v_mov_b32_e32 v7, 2", "v_mov_b32_e32 v140, 2")) == []
    assert run(good.replace("v_mov_b32_e32 v8, 3", "v_mov_b32_e32 v150, 3")) == []
    assert any("assembly names" in b for b in run(good.replace("v[136:137]", "v[0xa6:0xa9]")))
    assert any("scratch" in b for b in run(good, log.replace("ScratchSize [bytes/lane]: 0", "ScratchSize [bytes/lane]: 16")))
    assert any("register count" in b for b in run(good, log.replace("VGPRs: 168", "VGPRs: 124")))
    assert any("do not fit" in b for b in run(good, log.replace("Occupancy [waves/SIMD]: 3", "Occupancy [waves/SIMD]: 2")))
    # an access through a generic address, anywhere in the kernel (an LDS offset of 0 turned into a
    # generic pointer is the null pointer: the access goes to global address 0)
    assert any("generic address" in b for b in run(good.replace("v_mov_b32_e32 v8, 3", "flat_store_dword v[2:3], v1 sc0 sc1")))
    assert any("generic address" in b for b in run(good.replace("v_mov_b32_e32 v7, 2", "flat_load_dword v1, v[2:3]")))


def test_a_spilling_instance_of_a_wait_counting_kernel_is_refused():
    """the build reads every unit's resource remarks: scratch memory in a kernel that waits for its
    own copies by count is a reason not to link, in any other kernel it is not"""
    remark = ("remark: Function Name: %s\nremark:     VGPRs: 128\nremark:     AGPRs: 0\n"
              "remark:     ScratchSize [bytes/lane]: %d\nremark:     Occupancy [waves/SIMD]: 4\n")
    tn = "_ZN4amos12amos_gemm_tnILi0ELi256ELi256ELi2ELi2ELi3EEEvNS_12GemmTnParamsE"
    other = "_ZN4amos10amos_igemmILi0ELi0ELi0ELi1ELi1EEEvNS_11IgemmParamsE"
    assert isa_check.spills("x", remark % (tn, 0) + remark % (other, 24)) == []
    bad = isa_check.spills("x", remark % (tn, 24) + remark % (other, 0))
    assert len(bad) == 1 and "amos_gemm_tn" in bad[0] and "24 bytes" in bad[0]
    for k in ("_ZN4amos15amos_conv_fpropILi0EEEvNS_15ConvFpropParamsE", "_ZN4amos14amos_conv_nchwILi0EEEvNS_14ConvNchwParamsE"):
        assert len(isa_check.spills("x", remark % (k, 8))) == 1
