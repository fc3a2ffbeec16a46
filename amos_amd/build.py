"""Builds libamos_mi355x.so for gfx950 with hipcc:  python -m amos_amd.build"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libamos_mi355x.so")

# -packed-fp32-ops is switched off: the compiler must not form v_pk_*_f32
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
# AMOS_BUILD_SPLIT_IN_KERNEL=1 in the environment of the build compiles the split-K tails into the
# kernels (igemm_kernel.h: split_finish); the default library does not have them
if os.environ.get("AMOS_BUILD_SPLIT_IN_KERNEL") == "1":
    HIP_FLAGS.append("-DAMOS_SPLIT_IN_KERNEL=1")


def sources():
    hip = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    cpp = sorted(f for f in os.listdir(CSRC) if f.endswith(".cpp"))
    return [os.path.join(CSRC, f) for f in hip + cpp]


def build(verbose=True, jobs=8):
    """compile every translation unit (in parallel), read the compiled code of the kernels whose
    assembly statements own registers (isa_check) and link the shared library only if that holds"""
    from . import isa_check
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs, objs = [], []
    jobs_list = []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        objs.append(obj)
        remarks = ["-Rpass-analysis=kernel-resource-usage"] if src.endswith(".hip") else []
        jobs_list.append((src, obj, [hipcc] + HIP_FLAGS + inc + remarks + ["-c", src, "-o", obj]))
    # the same units once more as assembly text, for the check
    checked = []
    for unit in isa_check.UNITS:
        src = os.path.join(CSRC, unit)
        asm = os.path.join(objdir, unit + ".s")
        checked.append((unit, asm))
        jobs_list.append((src, asm, [hipcc] + HIP_FLAGS + inc + isa_check.ASM_FLAGS + [src, "-o", asm]))
    for src, out, cmd in jobs_list:
        if verbose:
            print(" ".join(cmd), flush=True)
        # (the compiler's output goes to a file: a pipe that nobody reads while we wait for the
        # process fills up after 64 KB of diagnostics and the compiler then blocks for good)
        log = open(out + ".log", "w+b")
        procs.append((src, out, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT), log))
        while sum(p.poll() is None for _, _, p, _ in procs) >= jobs:
            for _, _, p, _ in procs:
                if p.poll() is None:
                    p.wait()
                    break
    logs = {}
    for src, out, p, log in procs:
        p.wait()
        log.seek(0)
        text = log.read().decode()
        log.close()
        logs[out] = text
        shown = "\n".join(l for l in text.splitlines() if "packed-fp32-ops" not in l and "remark:" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, shown))
        if verbose and shown.strip() and not out.endswith(".s"):   # (the assembly jobs' output is remarks)
            print(shown)
    bad = []
    for unit, asm in checked:
        bad += isa_check.violations(unit, asm, logs[asm])[1]
    # kernels that count their own memory waits must not spill: scratch traffic uses the same counter
    for obj in objs:
        bad += isa_check.spills(os.path.basename(obj), logs[obj])
    if bad:
        if os.path.exists(OUT):
            os.remove(OUT)
        raise RuntimeError("not linking %s: the compiled code breaks the rule of amos_amd/isa_check.py\n%s"
                           % (OUT, "\n".join(bad)))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build()
    sys.exit(0)
