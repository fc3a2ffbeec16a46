"""Reads the compiled code of the NCDHW-direct convolution instances (csrc/conv_nchw_kernel.h).

Their loader waves keep global loads in flight across the loop's back edge in registers that only
their assembly statements name: the 32 highest registers a wave of the workgroup's size can have
(v136..v167 with twelve waves per compute unit, v224..v255 with eight).  That is sound only while
nothing the compiler generates touches those registers: an address the compiler keeps there
would be overwritten by a load that lands, and the next access through it faults.  So the build
refuses to link a library, and a test fails, unless for every instance

  * no instruction outside the assembly statements names a staging register;
  * the assembly statements stay inside the 32 staging registers;
  * the instance neither spills to scratch memory nor uses accumulation registers, its register
    count covers the staging registers and leaves room for the waves of one workgroup on a
    compute unit.
"""
import re

UNITS = ["inst_conv_nchw_f16.hip", "inst_conv_nchw_bf16.hip", "inst_conv_nchw_i8.hip"]
ASM_FLAGS = ["-S", "--cuda-device-only", "-Rpass-analysis=kernel-resource-usage"]
_NUM = r"(0x[0-9a-fA-F]+|\d+)"
_VREG = re.compile(r"\bv(\d+)\b|\bv\[" + _NUM + r"(?::" + _NUM + r")?\]")


def vregs(text):
    """the vector registers an instruction's text names"""
    out = set()
    for m in _VREG.finditer(text):
        if m.group(1) is not None:
            out.add(int(m.group(1)))
        else:
            a = int(m.group(2), 0)
            b = int(m.group(3), 0) if m.group(3) else a
            out.update(range(a, b + 1))
    return out


def instances(asm_path):
    """{kernel symbol: {targs, waves, base (first staging register), outside: instructions outside
    assembly statements that name a staging register, inside: staging registers the assembly
    statements name}}"""
    found, name, inasm = {}, None, False
    for line in open(asm_path):
        m = re.match(r"^(_ZN4amos14amos_conv_nchw\w+):", line)
        if m:
            name = m.group(1)
            t = [int(x) for x in re.findall(r"Li(\d+)E", name)]
            waves = t[3] * t[4] + t[7]          # WI * WJ matrix-core waves + NWL loader waves
            found[name] = {"targs": t, "waves": waves, "base": {12: 136, 8: 224}.get(waves, -1), "outside": [], "inside": set()}
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
        high = {r for r in vregs(code) if r >= rec["base"]}
        if inasm:
            rec["inside"] |= high
        elif high:
            rec["outside"].append(code)
    return found


def resources(log_text):
    """{kernel symbol: {vgprs, agprs, scratch, occupancy}} from the compiler's resource remarks"""
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


def violations(unit, asm_path, log_text):
    """(number of instances read, [what is wrong]) for one translation unit"""
    bad = []
    inst = instances(asm_path)
    res = resources(log_text)
    if not inst:
        bad.append("%s: no amos_conv_nchw instance" % unit)
    for name, rec in inst.items():
        what = "%s %s" % (unit, rec["targs"])
        if rec["base"] < 0:
            bad.append("%s: a workgroup of %d waves has no staging registers assigned" % (what, rec["waves"]))
            continue
        if rec["outside"]:
            bad.append("%s: compiler-generated code names a staging register: %s" % (what, rec["outside"][:3]))
        if not rec["inside"]:
            bad.append("%s: no staging register in its assembly statements" % what)
            continue
        if max(rec["inside"]) >= rec["base"] + 32:
            bad.append("%s: assembly names v%d" % (what, max(rec["inside"])))
        r = res.get(name)
        if r is None:
            bad.append("%s: no resource remarks" % what)
            continue
        if r.get("scratch", 0) or r.get("agprs", 0):
            bad.append("%s: scratch memory or accumulation registers: %s" % (what, r))
        # (the wave's register allocation covers the staging registers, and nothing above them)
        if not max(rec["inside"]) < r.get("vgprs", 0) <= rec["base"] + 32:
            bad.append("%s: register count %s" % (what, r))
        if r.get("occupancy", 0) * 4 < rec["waves"]:
            bad.append("%s: %d waves do not fit (%s)" % (what, rec["waves"], r))
    return len(inst), bad
