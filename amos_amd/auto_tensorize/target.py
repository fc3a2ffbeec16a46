"""Target descriptor of the MI355X (replaces python/tvm/auto_tensorize/target.py:56-88, the
per-architecture limits of `CUDA(arch)`)."""

supported_target = ["hip", "rocm"]


class AcceleratorTarget(object):
    pass


class MI355X(AcceleratorTarget):
    """gfx950: 256 CUs in 8 XCDs, 64-lane wavefronts, 160 KB LDS per CU, 512 registers per lane
    (VGPR + AGPR) at one wave per SIMD, 288 GB HBM3E"""

    arch = "gfx950"

    def get_shared_memory_bytes(self): return 160 * 1024
    def get_warp_size(self): return 64
    def get_register_bytes_per_thread(self): return 512 * 4
    def max_threads(self): return 1024
    def max_blocks(self): return 2 ** 31 - 1
    def compute_units(self): return 256
    def peak_tflops(self, dtype): return 5033.2 if dtype == "int8" else 2516.6
    def hbm_bytes_per_second(self): return 8e12


def get_device_arch(dev_id=0):
    """arch string of the device (replaces get_cuda_compute_version, target.py:27-49)"""
    from .. import ops
    return ops.device_info().arch.decode().split(":")[0]
