"""Reads the compiled code of the NCDHW-direct convolution instances (csrc/conv_nchw_kernel.h).

Their loader waves keep global loads in flight across the loop's back edge in registers that only
their assembly statements name: the 32 highest registers a wave of the workgroup's size can have
(v136..v167 with twelve waves per compute unit, v224..v255 with eight).  That is sound only while
nothing the compiler generates touches those registers: an address the compiler keeps there
would be overwritten by a load that lands, and the next access through it faults.  So the build
refuses to link a library, and a test fails, unless for every instance

  * no compiler-generated instruction names a staging register between a staging load and the wait
    for it: followed along the kernel's labels and branches from every assembly statement that
    loads into a staging register up to the next assembly statement `s_waitcnt vmcnt(0)` -- the
    stretch in which the data lands.  (A value the compiler keeps across a staging load cannot sit
    in one of these registers: the load statements declare them clobbered.  Code outside those
    stretches -- the matrix-core waves' in particular, other waves with registers of their own --
    may use every register the workgroup size leaves it.)
  * the assembly statements stay inside the 32 staging registers;
  * the instance neither spills to scratch memory nor uses accumulation registers, its register
    count covers the staging registers and leaves room for the waves of one workgroup on a
    compute unit;
  * no instruction accesses memory through a generic ("flat") address: the kernel names global
    memory and the LDS in their own address spaces.  (An LDS byte offset turned into a generic
    pointer is what this catches: the compiler folds offset 0 into the null pointer, and the
    access becomes one of global address 0 -- a memory fault.)
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


_LABEL = re.compile(r"^(\.LBB\d+_\d+):")
_BRANCH = re.compile(r"^\s*(s_branch|s_cbranch_\w+)\s+(\.LBB\d+_\d+)")


def _blocks(lines):
    """basic blocks of one kernel's assembly text: [{label, code: [(text, inside an assembly
    statement)], succ: [block indices]}]"""
    blocks, cur, inasm = [], {"label": None, "code": [], "targets": [], "falls": True}, False
    for line in lines:
        m = _LABEL.match(line)
        if m:
            blocks.append(cur)
            cur = {"label": m.group(1), "code": [], "targets": [], "falls": True}
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
        if not cur["falls"]:   # code behind an unconditional branch without a label: its own block
            blocks.append(cur)
            cur = {"label": None, "code": [], "targets": [], "falls": True}
        cur["code"].append((code, inasm))
        b = _BRANCH.match(code)
        if b:
            cur["targets"].append(b.group(2))
            if b.group(1) == "s_branch":
                cur["falls"] = False
        elif code.startswith("s_endpgm"):
            cur["falls"] = False
    blocks.append(cur)
    index = {b["label"]: i for i, b in enumerate(blocks) if b["label"]}
    for i, b in enumerate(blocks):
        b["succ"] = [index[t] for t in b["targets"] if t in index]
        if b["falls"] and i + 1 < len(blocks):
            b["succ"].append(i + 1)
    return blocks


def instances(asm_path):
    """{kernel symbol: {targs, waves, base (first staging register), outside: compiler-generated
    instructions between a staging load and its wait that name a staging register, inside: staging
    registers the assembly statements name}}"""
    found, name, body = {}, None, []

    def finish():
        rec = found[name]
        base = rec["base"]
        blocks = _blocks(body)
        index = {b["label"]: i for i, b in enumerate(blocks) if b["label"]}
        is_load = lambda code, inasm: inasm and "load" in code and any(r >= base for r in vregs(code))
        is_wait = lambda code, inasm: inasm and code.replace(" ", "") == "s_waitcntvmcnt(0)"
        for b in blocks:
            for code, inasm in b["code"]:
                if inasm:
                    rec["inside"] |= {r for r in vregs(code) if r >= base}
                if re.match(r"flat_(load|store|atomic)", code):
                    rec["flat"].append(code)
        # from behind every staging load, forward until the wait
        seen_block_starts, todo, flagged = set(), [], []
        for i, b in enumerate(blocks):
            for k, (code, inasm) in enumerate(b["code"]):
                if is_load(code, inasm):
                    todo.append((i, k + 1))
        done = set()
        while todo:
            i, k = todo.pop()
            if (i, k) in done:
                continue
            done.add((i, k))
            stopped = False
            follow = []
            for code, inasm in blocks[i]["code"][k:]:
                if is_wait(code, inasm):
                    stopped = True
                    break
                if not inasm and any(r >= base for r in vregs(code)):
                    flagged.append(code)
                b = _BRANCH.match(code)
                if b and b.group(2) in index:      # a branch in front of the wait leaves the block
                    follow.append(index[b.group(2)])
            if not stopped:
                follow = blocks[i]["succ"]
            for j in follow:
                if j not in seen_block_starts:
                    seen_block_starts.add(j)
                    todo.append((j, 0))
        rec["outside"] = flagged

    for line in open(asm_path):
        m = re.match(r"^(_ZN4amos14amos_conv_nchw\w+):", line)
        if m:
            name = m.group(1)
            t = [int(x) for x in re.findall(r"Li(\d+)E", name)]
            waves = t[3] * t[4] + t[7]          # WI * WJ matrix-core waves + NWL loader waves
            found[name] = {"targs": t, "waves": waves, "base": {12: 136, 8: 224}.get(waves, -1), "outside": [], "inside": set(), "flat": []}
            body = []
            continue
        if name is None:
            continue
        if line.startswith(".Lfunc_end"):
            finish()
            name = None
            continue
        body.append(line)
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


# Kernels whose pipelines wait for their own global -> LDS copies and global loads by count
# (s_waitcnt vmcnt(n), n > 0): a register spill's scratch access counts on the same counter, so a
# spilling instance would wait for the wrong accesses.  The build refuses such an instance; the
# library refuses to launch one as well (amos_runtime.hip: launch_tn, launch_conv).
NO_SCRATCH = ("amos_gemm_tn", "amos_conv_fprop", "amos_conv_nchw")


def spills(unit, log_text):
    """[what is wrong] for one translation unit's resource remarks"""
    bad = []
    for name, r in resources(log_text).items():
        if any(("%d%s" % (len(k), k)) in name for k in NO_SCRATCH) and r.get("scratch", 0):
            bad.append("%s: %s spills %d bytes per lane to scratch memory" % (unit, name, r["scratch"]))
    return bad


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
        if rec["flat"]:
            bad.append("%s: memory accessed through a generic address: %s" % (what, rec["flat"][:3]))
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
