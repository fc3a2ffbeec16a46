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


def sources():
    hip = sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))
    cpp = sorted(f for f in os.listdir(CSRC) if f.endswith(".cpp"))
    return [os.path.join(CSRC, f) for f in hip + cpp]


def build(verbose=True, jobs=8):
    """compile every translation unit (in parallel) and link the shared library"""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC]
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    procs, objs = [], []
    for src in sources():
        obj = os.path.join(objdir, os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = [hipcc] + HIP_FLAGS + inc + ["-c", src, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        # (the compiler's output goes to a file: a pipe that nobody reads while we wait for the
        # process fills up after 64 KB of diagnostics and the compiler then blocks for good)
        log = open(obj + ".log", "w+b")
        procs.append((src, subprocess.Popen(cmd, stdout=log, stderr=subprocess.STDOUT), log))
        while sum(p.poll() is None for _, p, _ in procs) >= jobs:
            for _, p, _ in procs:
                if p.poll() is None:
                    p.wait()
                    break
    for src, p, log in procs:
        p.wait()
        log.seek(0)
        out = log.read()
        log.close()
        text = "\n".join(l for l in out.decode().splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError("hipcc failed on %s:\n%s" % (src, text))
        if verbose and text.strip():
            print(text)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", OUT]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return OUT


if __name__ == "__main__":
    build()
    sys.exit(0)
