"""ctypes binding of libamos_mi355x.so (C ABI declared in include/amos_mi355x.h)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libamos_mi355x.so")

AMOS_F16, AMOS_BF16, AMOS_I8, AMOS_F32, AMOS_I32 = range(5)
AMOS_OP_GEMM, AMOS_OP_BGEMM, AMOS_OP_CONV2D, AMOS_OP_CONV3D = range(4)

AMOS_PIPE_AUTO, AMOS_PIPE_STAGED, AMOS_PIPE_DIRECT4, AMOS_PIPE_DIRECT8, AMOS_PIPE_PATCH, AMOS_PIPE_PATCH8, AMOS_PIPE_NCHW = range(7)

AMOS_ERR_BAD_ARG = -1
AMOS_ERR_UNSUPPORTED = -2
AMOS_ERR_INFEASIBLE = -3
AMOS_ERR_HIP = -4
AMOS_ERR_WORKSPACE = -5
AMOS_NOALLOC_SCRATCH_BYTES = 8 << 20

DTYPE_CODE = {"float16": AMOS_F16, "bfloat16": AMOS_BF16, "int8": AMOS_I8, "float32": AMOS_F32,
              "int32": AMOS_I32}

_i32, _i64 = ctypes.c_int32, ctypes.c_int64


class DeviceInfo(ctypes.Structure):
    _fields_ = [("compute_units", _i32), ("wave_size", _i32), ("max_clock_khz", _i32),
                ("lds_bytes_per_block", _i32), ("hbm_bytes", _i64), ("arch", ctypes.c_char * 64),
                ("peak_tflops_f16", ctypes.c_double), ("peak_tops_i8", ctypes.c_double)]


class GemmDesc(ctypes.Structure):
    _fields_ = [("M", _i64), ("N", _i64), ("K", _i64), ("in_dtype", _i32), ("out_dtype", _i32),
                ("trans_a", _i32), ("trans_b", _i32), ("lda", _i64), ("ldb", _i64), ("ldc", _i64)]


class BGemmDesc(ctypes.Structure):
    _fields_ = [("batch", _i64), ("g", GemmDesc), ("stride_a", _i64), ("stride_b", _i64),
                ("stride_c", _i64)]


class ConvDesc(ctypes.Structure):
    _fields_ = [("N", _i64), ("C", _i64), ("D", _i64), ("H", _i64), ("W", _i64), ("K", _i64),
                ("T", _i64), ("R", _i64), ("S", _i64),
                ("stride_d", _i32), ("stride_h", _i32), ("stride_w", _i32),
                ("pad_d", _i32), ("pad_h", _i32), ("pad_w", _i32),
                ("dil_d", _i32), ("dil_h", _i32), ("dil_w", _i32),
                ("in_dtype", _i32), ("out_dtype", _i32), ("groups", _i32), ("layout", _i32)]


class KernelConfig(ctypes.Structure):
    _fields_ = [("tile_i", _i32), ("tile_j", _i32), ("split_k", _i32), ("pipeline", _i32),
                ("reserved", _i32 * 4)]


AMOS_EPI_NONE, AMOS_EPI_ADD = 0, 1
AMOS_LAYOUT_NCHW, AMOS_LAYOUT_NHWC, AMOS_LAYOUT_HWNC = 0, 1, 2
LAYOUT_CODE = {"nchw": 0, "ncdhw": 0, "nhwc": 1, "ndhwc": 1, "hwnc": 2, "dhwnc": 2}
AMOS_FLAG_NO_UNROLLED_TAPS, AMOS_FLAG_NO_TILE_WALK, AMOS_FLAG_WEIGHTS_PACKED = 1, 2, 4


class Epilogue(ctypes.Structure):
    _fields_ = [("kind", _i32), ("dtype", _i32), ("operand", ctypes.c_void_p), ("ld", _i64),
                ("stride", _i64)]


class GatherDesc(ctypes.Structure):
    _fields_ = [("ndim", _i32), ("elem_bytes", _i32), ("out_shape", _i64 * 5), ("table_offset", _i64 * 5),
                ("in_elems", _i64)]


AMOS_ELT_LOAD, AMOS_ELT_CONST, AMOS_ELT_ADD, AMOS_ELT_SUB, AMOS_ELT_MUL = 1, 2, 3, 4, 5


class EltwiseDesc(ctypes.Structure):
    _fields_ = [("dtype", _i32), ("n_inputs", _i32), ("n_ops", _i32), ("reserved", _i32), ("elems", _i64),
                ("program", _i32 * 16), ("consts", ctypes.c_float * 4)]


class ComputeC(ctypes.Structure):
    _fields_ = [("n_tokens", _i32), ("tokens", ctypes.POINTER(_i32)), ("n_iters", _i32),
                ("iter_kinds", ctypes.POINTER(_i32)), ("iter_extents", ctypes.POINTER(_i64)),
                ("n_loads", _i32), ("load_ndim", ctypes.POINTER(_i32)),
                ("coeffs", ctypes.POINTER(_i64))]


class AmosError(RuntimeError):
    """A C-ABI call returned a negative code; `.code` holds it."""

    def __init__(self, code, msg):
        super().__init__("libamos_mi355x error %d: %s" % (code, msg))
        self.code = code


# every symbol include/amos_mi355x.h declares
EXPORTS = [
    "amos_version", "amos_last_error", "amos_device_info", "amos_default_config",
    "amos_check_config", "amos_workspace_bytes", "amos_estimate_seconds", "amos_gemm", "amos_bgemm", "amos_conv2d",
    "amos_conv3d", "amos_conv2d_noalloc", "amos_conv_packed_weights_bytes", "amos_conv_pack_weights", "amos_run_fused", "amos_time", "amos_time_fused", "amos_gather", "amos_time_gather",
    "amos_eltwise", "amos_time_eltwise", "amos_kernel_name", "amos_match", "amos_enumerate_mappings",
    "amos_mfma_ceiling",
]

_lib = None


def load():
    """Load the shared library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with `python -m amos_amd.build` (hipcc, gfx950)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    vp, sz = ctypes.c_void_p, ctypes.c_size_t
    lib.amos_version.restype = ctypes.c_int
    lib.amos_last_error.restype = ctypes.c_char_p
    lib.amos_device_info.argtypes = [ctypes.POINTER(DeviceInfo)]
    lib.amos_default_config.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig)]
    lib.amos_check_config.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig),
                                      ctypes.POINTER(_i64), ctypes.POINTER(_i64)]
    lib.amos_workspace_bytes.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig)]
    lib.amos_workspace_bytes.restype = sz
    lib.amos_estimate_seconds.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig),
                                          ctypes.POINTER(ctypes.c_double)]
    for name, desc in (("amos_gemm", GemmDesc), ("amos_bgemm", BGemmDesc), ("amos_conv2d", ConvDesc),
                       ("amos_conv3d", ConvDesc)):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.POINTER(desc), ctypes.POINTER(KernelConfig), vp, vp, vp, vp, sz, vp]
        fn.restype = ctypes.c_int
    lib.amos_conv_packed_weights_bytes.argtypes = [ctypes.c_int, ctypes.POINTER(ConvDesc)]
    lib.amos_conv_packed_weights_bytes.restype = sz
    lib.amos_conv_pack_weights.argtypes = [ctypes.c_int, ctypes.POINTER(ConvDesc), vp, vp, vp]
    lib.amos_conv_pack_weights.restype = ctypes.c_int
    lib.amos_conv2d_noalloc.argtypes = [ctypes.POINTER(ConvDesc), ctypes.POINTER(KernelConfig), vp, vp, vp, vp]
    lib.amos_conv2d_noalloc.restype = ctypes.c_int
    lib.amos_time.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig), vp, vp, vp, vp, sz, vp,
                              ctypes.c_int, ctypes.c_int, ctypes.c_int,
                              ctypes.POINTER(ctypes.c_double)]
    lib.amos_run_fused.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig), ctypes.POINTER(Epilogue),
                                   vp, vp, vp, vp, sz, vp]
    lib.amos_time_fused.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig), ctypes.POINTER(Epilogue),
                                    vp, vp, vp, vp, sz, vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                    ctypes.POINTER(ctypes.c_double)]
    lib.amos_mfma_ceiling.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, sz, vp,
                                      ctypes.c_int, vp, ctypes.POINTER(ctypes.c_double),
                                      ctypes.POINTER(ctypes.c_double)]
    lib.amos_mfma_ceiling.restype = ctypes.c_int
    lib.amos_gather.argtypes = [ctypes.POINTER(GatherDesc), vp, vp, vp, vp]
    lib.amos_eltwise.argtypes = [ctypes.POINTER(EltwiseDesc), ctypes.POINTER(vp), vp, vp]
    lib.amos_eltwise.restype = ctypes.c_int
    lib.amos_time_eltwise.argtypes = [ctypes.POINTER(EltwiseDesc), ctypes.POINTER(vp), vp, vp, ctypes.c_int,
                                      ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.amos_time_eltwise.restype = ctypes.c_int
    lib.amos_time_gather.argtypes = [ctypes.POINTER(GatherDesc), vp, vp, vp, vp, ctypes.c_int, ctypes.c_int,
                                     ctypes.c_int, ctypes.POINTER(ctypes.c_double)]
    lib.amos_kernel_name.argtypes = [ctypes.c_int, vp, ctypes.POINTER(KernelConfig)]
    lib.amos_kernel_name.restype = ctypes.c_char_p
    lib.amos_match.argtypes = [ctypes.POINTER(ComputeC), ctypes.POINTER(ComputeC),
                               ctypes.POINTER(_i32), _i32]
    lib.amos_enumerate_mappings.argtypes = [_i32, _i32, ctypes.POINTER(_i32), ctypes.POINTER(_i64),
                                            ctypes.POINTER(_i64), ctypes.POINTER(ctypes.c_uint8),
                                            ctypes.POINTER(ctypes.c_uint8), _i32]
    _lib = lib
    return lib


def check(rc):
    if rc < 0:
        raise AmosError(rc, load().amos_last_error().decode())
    return rc
