"""Hardware-abstraction DAGs (load -> mma -> store per dtype pair) and their registry.

Mirrors python/tvm/auto_tensorize/hw_abs_dag/hw_abs_dag_base.py (:91-305 base class,
:443-527 registry) with the CUDA entries of hw_abs_dag/cuda/wmma_fp16.py, wmma_bf16.py and
wmma_int8.py replaced by gfx950 MFMA entries.  Targets "hip" and "rocm" both resolve to them.
"""
from .hw_abstraction import (HW_ABS_REGISTER_POOL, InstructionScope, MFMA_INSTRUCTIONS,
                             compute_dag_from_tensors, mfma_fragment_layout)


class HardwareAbstractionDAG(object):
    target = None
    scope = InstructionScope.warp
    hw_abs_dict = {}
    edges = {}
    main_hw_abs_name = ""
    anchor_point = ""
    input_dtypes = {}
    output_dtypes = {}

    def get_name(self):
        raise NotImplementedError()

    def get_all_compute_keys(self):
        raise NotImplementedError()

    def get_all_shape_keys(self):
        raise NotImplementedError()

    def get_main_compute_expression(self, compute_key, shape_key):
        raise NotImplementedError()

    def get_effective_compute_dag(self, compute_key, shape_key):
        """(intrinsic ComputeDAG, main tensors) -- what the matcher compares a compute with
        (reference: hw_abs_dag_base.py:185-202)"""
        _, outs = self.get_main_compute_expression(compute_key, shape_key)
        return compute_dag_from_tensors(outs), outs

    def get_intrinsic(self, compute_key, shape_key, hw_abs_key=None):
        raise NotImplementedError()

    def get_header(self):
        return ""

    def get_special_dtype(self, dtype):
        return ""


class HwAbsDAGRegisterPool(object):
    def __init__(self):
        self.registries = {}

    def add(self, target, mnemonic, cls, override=False):
        self.registries.setdefault(target, {})
        if mnemonic in self.registries[target] and not override:
            raise RuntimeError("Try to add repeated hardware abstraction dag: target=%s, mnemonic=%s" % (target, mnemonic))
        self.registries[target][mnemonic] = cls

    def remove(self, target, mnemonic, allow_missing=False):
        if target not in self.registries or mnemonic not in self.registries[target]:
            if not allow_missing:
                raise RuntimeError("Try to remove missing hardware abstraction dag: target=%s, mnemonic=%s" % (target, mnemonic))
            return
        del self.registries[target][mnemonic]

    def find(self, target, mnemonic):
        if target not in self.registries or mnemonic not in self.registries[target]:
            return None
        return self.registries[target][mnemonic]

    def enumerate(self, target):
        return list(self.registries.get(target, {}).values())


HW_ABS_DAG_REGISTER_POOL = HwAbsDAGRegisterPool()


def register_hw_abs_dag(target, mnemonic, override=False):
    global HW_ABS_DAG_REGISTER_POOL

    def register(cls):
        HW_ABS_DAG_REGISTER_POOL.add(target, mnemonic, cls, override=override)
        return cls

    return register


def query_hw_abs_dag(target):
    """every DAG class registered for `target`, in registration order"""
    return HW_ABS_DAG_REGISTER_POOL.enumerate(str(target))


class MFMADag(HardwareAbstractionDAG):
    """load_a, load_b -> mma -> store on one wavefront"""
    target = "hip"
    scope = InstructionScope.warp
    mnemonic = None
    mma_mnemonic = None
    shape_keys = ()
    compute_keys = ("nnn", "ntn", "tnn", "ttn")
    edges = {"mma": ["load_a", "load_b"], "store": ["mma"]}
    main_hw_abs_name = "mma"
    anchor_point = "mma"

    def __init__(self):
        mma = HW_ABS_REGISTER_POOL.find("hip", self.mma_mnemonic)
        self.hw_abs_dict = {
            "load_a": HW_ABS_REGISTER_POOL.find("hip", "mfma::lds_load"),
            "load_b": HW_ABS_REGISTER_POOL.find("hip", "mfma::lds_load"),
            "mma": mma,
            "store": HW_ABS_REGISTER_POOL.find("hip", "mfma::global_store"),
        }
        self.mma = mma()
        self.input_dtypes = {"load_a": [self.mma.in_dtype], "load_b": [self.mma.in_dtype],
                             "mma": [self.mma.in_dtype, self.mma.in_dtype], "store": [self.mma.out_dtype]}
        self.output_dtypes = {"load_a": [self.mma.in_dtype], "load_b": [self.mma.in_dtype],
                              "mma": [self.mma.out_dtype], "store": [self.mma.out_dtype]}

    def get_name(self):
        return self.mnemonic

    def get_all_compute_keys(self):
        return list(self.compute_keys)

    def get_all_shape_keys(self):
        return list(self.shape_keys)

    def get_problem_size(self, shape_key):
        return [int(x) for x in shape_key.split("x")]

    def get_main_compute_expression(self, compute_key, shape_key):
        """compute key = transposition of (A, B, C): 'n' row-major, 't' column-major"""
        m, n, k = self.get_problem_size(shape_key)
        tA, tB, tC = (ch == "t" for ch in compute_key)
        a_shape = (k, m) if tA else (m, k)
        b_shape = (n, k) if tB else (k, n)
        return self.mma.get_compute_expression([a_shape, b_shape], (m, n), tA, tB, tC)

    def get_intrinsic(self, compute_key, shape_key, hw_abs_key="mma"):
        return MFMA_INSTRUCTIONS[(self.mma.in_dtype, shape_key)]

    def get_fragment_layout(self, shape_key):
        return mfma_fragment_layout(shape_key)

    def get_memory_scope_realize(self, dtype, scope, constant_size, attributes):
        """operand fragments and accumulators are plain VGPR / AGPR arrays on gfx950"""
        return [None, constant_size]


def _register_both(mnemonic):
    def deco(cls):
        cls.mnemonic = mnemonic
        register_hw_abs_dag("hip", mnemonic)(cls)
        register_hw_abs_dag("rocm", mnemonic)(cls)
        return cls
    return deco


@_register_both("mfma_f16_f32")
class MFMAFp16Fp32(MFMADag):
    mma_mnemonic = "mfma_f16_f32::mma"
    shape_keys = ("32x32x16", "16x16x32")


@_register_both("mfma_bf16_f32")
class MFMABf16Fp32(MFMADag):
    mma_mnemonic = "mfma_bf16_f32::mma"
    shape_keys = ("32x32x16", "16x16x32")


@_register_both("mfma_i8_i32")
class MFMAInt8Int32(MFMADag):
    mma_mnemonic = "mfma_i8_i32::mma"
    shape_keys = ("32x32x32", "16x16x64")


@_register_both("mfma_i8_i32_wrapped_spelling")
class MFMAInt8Int32WrappedSpelling(MFMADag):
    """accepts (a * b).astype("int32") on int8 operands; see MFMAI8I32MmaWrappedSpelling"""
    mma_mnemonic = "mfma_i8_i32::mma_wrapped_spelling"
    shape_keys = ("32x32x32", "16x16x64")
    wrapped_spelling = True


class MFMABiasDag(MFMADag):
    """load_a, load_b -> mma, load_bias -> bias -> store: the DAG with an element-wise stage
    behind the MMA.  Like the reference's WMMAFp16Fp32Bias (hw_abs_dag/cuda/wmma_fp16_bias.py:11-56)
    it is NOT registered: query_hw_abs_dag() and the matching counts of the tutorial flow do not
    see it.  A compute with such a tail still matches the plain DAG on its main op, and lowering
    fuses the tail into the kernel (lowering.py)."""
    edges = {"mma": ["load_a", "load_b"], "bias": ["mma", "load_bias"], "store": ["bias"]}
    anchor_point = "bias"
    bias_dtype = None

    def __init__(self):
        super().__init__()
        self.hw_abs_dict = dict(self.hw_abs_dict)
        self.hw_abs_dict["load_bias"] = HW_ABS_REGISTER_POOL.find("hip", "mfma::lds_load")
        self.hw_abs_dict["bias"] = HW_ABS_REGISTER_POOL.find("hip", "mfma::add_bias")
        self.input_dtypes = dict(self.input_dtypes, load_bias=[self.bias_dtype],
                                 bias=[self.mma.out_dtype, self.bias_dtype], store=[self.mma.out_dtype])
        self.output_dtypes = dict(self.output_dtypes, load_bias=[self.bias_dtype], bias=[self.mma.out_dtype])

    def get_effective_compute_dag(self, compute_key, shape_key):
        """two ops: the MMA (op_lst[0]) and the element-wise addition behind it (op_lst[1])"""
        _, outs = self.get_main_compute_expression(compute_key, shape_key)
        m, n, _ = self.get_problem_size(shape_key)
        shape = [int(x) for x in outs[0].shape]
        _, tail = self.hw_abs_dict["bias"]().get_compute_expression_with_inputs(
            [outs[0]], [shape, shape], [shape], [self.mma.out_dtype, self.bias_dtype], [self.mma.out_dtype])
        return compute_dag_from_tensors(tail), outs


class MFMAFp16Fp32Bias(MFMABiasDag):
    mnemonic = "mfma_f16_f32_bias"
    mma_mnemonic = "mfma_f16_f32::mma"
    shape_keys = ("32x32x16", "16x16x32")
    bias_dtype = "float16"


class MFMAInt8Int32Bias(MFMABiasDag):
    mnemonic = "mfma_i8_i32_bias"
    mma_mnemonic = "mfma_i8_i32::mma"
    shape_keys = ("32x32x32", "16x16x64")
    bias_dtype = "int32"
