"""bench.py's contract, as far as it can be checked without a GPU: more than one GPU is refused
with a message, and the counter summaries under profiles/ still describe the kernels as built --
each summary carries a hash of the kernel sources it was measured on, and bench.py reports
`roofline.traffic` / `traffic_bytes` from it only while that hash matches (a kernel edited after
its counters were taken must be profiled again)."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert p.returncode != 0 and "one-GPU" in (p.stderr + p.stdout)


def test_counter_summaries_match_the_kernel_sources():
    sys.path.insert(0, ROOT)
    import bench
    from amos_amd import _lib, ops
    import torch
    configs = {
        "C2": (_lib.AMOS_OP_GEMM, ops.gemm_desc(8192, 8192, 8192, torch.float16, False, True)),
        "C3": (_lib.AMOS_OP_CONV2D, ops.conv_desc((32, 256, 1, 14, 14), (256, 256, 1, 3, 3), torch.float16, (1, 1, 1), (0, 1, 1), (1, 1, 1))),
        "C4": (_lib.AMOS_OP_CONV2D, ops.conv_desc((64, 128, 1, 28, 28), (128, 128, 1, 3, 3), torch.int8, (1, 1, 1), (0, 1, 1), (1, 1, 1))),
        "C5a": (_lib.AMOS_OP_BGEMM, ops.bgemm_desc(192, 512, 512, 64, torch.float16, False, True)),
        "C5b": (_lib.AMOS_OP_CONV3D, ops.conv_desc((8, 64, 16, 56, 56), (64, 64, 3, 3, 3), torch.float16, (1, 1, 1), (1, 1, 1), (1, 1, 1))),
    }
    stale = bench.stale_summaries()
    for name, (op, desc) in configs.items():
        kernel = ops.kernel_name(op, desc)      # the default configuration's kernel, as bench.py runs it
        traffic = bench.measured_traffic(kernel)
        if traffic is None and name != "C2":
            # A kernel that changed after its counters were read and could not be profiled again:
            # the summary must say so, naming the kernel that ships now (bench.py then reports no
            # traffic for it).  The headline kernel (roofline.traffic) has no such way out.
            assert name in stale and stale[name]["kernel_now"] == kernel and stale[name]["why"], \
                "%s: neither a current counter summary nor a stale_json line for %s" % (name, kernel)
            continue
        assert traffic is not None and traffic > 0, "%s: no current counter summary for %s" % (name, kernel)
