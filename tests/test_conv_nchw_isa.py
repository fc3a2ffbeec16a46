"""The loader waves of the NCDHW-direct convolution (csrc/conv_nchw_kernel.h) keep global loads in
flight across the loop's back edge in registers that only their assembly statements name: the 32
highest registers a wave of the workgroup's size can have (v136..v167 with twelve waves per compute
unit, v224..v255 with eight).  That is sound only while nothing the compiler generates touches
those registers.  This test compiles every instance to assembly (no GPU needed) and reads it:

  * outside the assembly statements no instruction names a staging register;
  * the assembly statements stay inside the 32 staging registers;
  * no instance spills to scratch memory or uses accumulation registers; its register count
    covers the staging registers and leaves room for the waves of one workgroup on a compute unit.
"""
import os
import re
import subprocess
import tempfile

import pytest

from amos_amd import build as amos_build

UNITS = ["inst_conv_nchw_f16.hip", "inst_conv_nchw_bf16.hip", "inst_conv_nchw_i8.hip"]
NUM = r"(0x[0-9a-fA-F]+|\d+)"
VREG = re.compile(r"\bv(\d+)\b|\bv\[" + NUM + r"(?::" + NUM + r")?\]")


def _vregs(text):
    out = set()
    for m in VREG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            a = int(m.group(2), 0)
            b = int(m.group(3), 0) if m.group(3) else a
            out.update(range(a, b + 1))
    return out


def _compile_all(tmp):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    procs = []
    for u in UNITS:
        out = os.path.join(tmp, u + ".s")
        log = open(os.path.join(tmp, u + ".log"), "w+")
        cmd = [hipcc] + amos_build.HIP_FLAGS + ["-I" + os.path.join(amos_build.ROOT, "include"), "-I" + amos_build.CSRC,
                                                "-S", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage",
                                                os.path.join(amos_build.CSRC, u), "-o", out]
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


def _instances(asm_path):
    """{kernel symbol: (template arguments, instructions outside assembly statements that name a
    staging register, staging registers the assembly statements name)}"""
    found, name, inasm = {}, None, False
    for line in open(asm_path):
        m = re.match(r"^(_ZN4amos14amos_conv_nchw\w+):", line)
        if m:
            name = m.group(1)
            t = [int(x) for x in re.findall(r"Li(\d+)E", name)]
            waves = t[3] * t[4] + t[7]          # WI * WJ matrix-core waves + NWL loader waves
            found[name] = {"targs": t, "waves": waves, "base": {12: 136, 8: 224}[waves], "outside": [], "inside": set()}
            continue
        if name is None:
            continue
        if line.startswith(".Lfunc_end"):
            name = None
            continue
        if "ASMSTART" in line:
            inasm = True
            continue
        if "ASMEND" in line:
            inasm = False
            continue
        code = line.split(";")[0].strip()
        if not code or code.startswith("."):
            continue
        rec = found[name]
        high = {r for r in _vregs(code) if r >= rec["base"]}
        if inasm:
            rec["inside"] |= high
        elif high:
            rec["outside"].append(code)
    return found


def _resources(log_text):
    rows, cur = {}, None
    for line in log_text.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            cur = rows.setdefault(m.group(1), {})
        for key, pat in (("agprs", r"AGPRs: (\d+)"), ("scratch", r"ScratchSize \[bytes/lane\]: (\d+)"),
                         ("occupancy", r"Occupancy \[waves/SIMD\]: (\d+)"), ("vgprs", r" VGPRs: (\d+)")):
            m = re.search(pat, line)
            if m and cur is not None:
                cur[key] = int(m.group(1))
    return rows


@pytest.mark.timeout(900)
def test_staging_registers_belong_to_the_assembly_statements():
    with tempfile.TemporaryDirectory() as tmp:
        built = _compile_all(tmp)
        total = 0
        for unit, asm, log in built:
            inst = _instances(asm)
            res = _resources(log)
            assert inst, "no amos_conv_nchw instance in %s" % unit
            for name, rec in inst.items():
                total += 1
                what = "%s %s" % (unit, rec["targs"])
                assert not rec["outside"], "%s: compiler-generated code names a staging register: %s" % (what, rec["outside"][:3])
                assert rec["inside"], "%s: no staging register in its assembly statements" % what
                assert max(rec["inside"]) < rec["base"] + 32, "%s: assembly names v%d" % (what, max(rec["inside"]))
                r = res.get(name)
                assert r is not None, "%s: no resource remarks" % what
                assert r.get("scratch", 0) == 0 and r.get("agprs", 0) == 0, "%s: %s" % (what, r)
                # (the wave's register allocation covers the staging registers, and nothing above them)
                assert max(rec["inside"]) < r["vgprs"] <= rec["base"] + 32, "%s: %s" % (what, r)
                assert r["occupancy"] * 4 >= rec["waves"], "%s: %d waves do not fit (%s)" % (what, rec["waves"], r)
        assert total >= 60
