"""Target descriptor of the MI355X (replaces python/tvm/auto_tensorize/target.py:56-88, the
per-architecture limits of `CUDA(arch)`)."""

supported_target = ["hip", "rocm"]

# MI355X's published dense peaks: the one place they are written down (bench.py and the reports
# divide by these; the figure a device's own clock and CU count give is amos_device_info's)
PEAK_F16_TFLOPS = 2500.0    # fp16 / bf16 MFMA, dense
PEAK_I8_TOPS = 5000.0       # int8 MFMA, dense
PEAK_HBM_GBS = 8000.0       # HBM3E


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
    def compute_units(self):
        """of the device when one is visible (a partitioned or binned part has fewer), else the full part's 256"""
        import torch
        if torch.cuda.is_available():
            from .. import ops
            return int(ops.device_info().compute_units)
        return 256

    def peak_tflops(self, dtype): return PEAK_I8_TOPS if dtype == "int8" else PEAK_F16_TFLOPS
    def hbm_bytes_per_second(self): return PEAK_HBM_GBS * 1e9


def get_device_arch(dev_id=0):
    """arch string of the device (replaces get_cuda_compute_version, target.py:27-49)"""
    from .. import ops
    return ops.device_info().arch.decode().split(":")[0]
