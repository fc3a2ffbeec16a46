"""Hardware abstractions: per-instruction descriptions of the CDNA4 (gfx950) matrix-core
path and the registry they live in.

Mirrors python/tvm/auto_tensorize/hw_abstraction/hw_abs_base.py (ComputeDAG :8-25, base
classes :28-202, register pool :205-287) with the Tensor Core WMMA entries
(hw_abstraction/cuda/wmma_base.py) replaced by v_mfma descriptions.  Where the reference's
classes emit CUDA text for the code generator, these carry the facts the hand-written
kernels are built on: operand fragment layouts, accumulator layout, LDS staging layout.
"""
from .. import te


class ComputeDAG(object):
    """Operations reachable from `tensors`, inputs first.
    (reference: src/auto_tensorize/hw_abstraction.cc:77-94, src/tg/graph/utils.cc:366-402)"""

    def __init__(self, tensors, op_lst, read_graph, feed_graph):
        self.tensors = list(tensors)
        self.op_lst = list(op_lst)
        self.read_graph = read_graph
        self.feed_graph = feed_graph

    def get_inputs(self):
        ret = []
        for op in self.op_lst:
            for inp in op.input_tensors:
                if isinstance(inp.op, te.PlaceholderOp):
                    ret.append(inp)
        return ret


def compute_dag_from_tensors(tensors):
    """ComputeOps in depth-first post-order from the root tensors; placeholders are not listed
    in op_lst but are keys of feed_graph."""
    op_lst, visited = [], set()
    read_graph, feed_graph = {}, {}

    def visit(op):
        if id(op) in visited:
            return
        visited.add(id(op))
        for inp in op.input_tensors:
            visit(inp.op)
            feed_graph.setdefault(inp.op, []).append(op)
        if isinstance(op, te.ComputeOp):
            read_graph[op] = [t.op for t in op.input_tensors]
            op_lst.append(op)

    for t in tensors:
        visit(t.op)
    return ComputeDAG(tensors, op_lst, read_graph, feed_graph)


class InstructionScope(object):
    warp = 0      # one 64-lane wavefront issues the instruction
    thread = 1


class HardwareAbstraction(object):
    target = None
    scope = InstructionScope.warp

    def get_name(self):
        return self.__class__.__name__

    def get_compute_expression(self, *args, **kwargs):
        raise NotImplementedError()

    def get_intrinsic(self, *args, **kwargs):
        raise NotImplementedError()


class MemoryAbstraction(HardwareAbstraction):
    pass


class ComputeAbstraction(HardwareAbstraction):
    pass


class ElementwiseComputeAbstraction(ComputeAbstraction):
    pass


class HardwareAbstractionRegisterPool(object):
    def __init__(self):
        self.registries = {}

    def add(self, target, mnemonic, cls, override=False):
        self.registries.setdefault(target, {})
        if mnemonic in self.registries[target] and not override:
            raise RuntimeError("Try to add repeated hardware abstraction: target=%s, mnemonic=%s" % (target, mnemonic))
        self.registries[target][mnemonic] = cls

    def remove(self, target, mnemonic, allow_missing=False):
        if target not in self.registries or mnemonic not in self.registries[target]:
            if not allow_missing:
                raise RuntimeError("Try to remove missing hardware abstraction: target=%s, mnemonic=%s" % (target, mnemonic))
            return
        del self.registries[target][mnemonic]

    def find(self, target, mnemonic):
        if target not in self.registries or mnemonic not in self.registries[target]:
            return None
        return self.registries[target][mnemonic]


HW_ABS_REGISTER_POOL = HardwareAbstractionRegisterPool()


def register_abstraction(target, mnemonic, override=False):
    global HW_ABS_REGISTER_POOL

    def register(cls):
        HW_ABS_REGISTER_POOL.add(target, mnemonic, cls, override=override)
        return cls

    return register


# ---- gfx950 v_mfma -----------------------------------------------------------------------
# instruction per (input dtype, shape key); shape keys are MxNxK of one issue
MFMA_INSTRUCTIONS = {
    ("float16", "32x32x16"): "v_mfma_f32_32x32x16_f16",
    ("float16", "16x16x32"): "v_mfma_f32_16x16x32_f16",
    ("bfloat16", "32x32x16"): "v_mfma_f32_32x32x16_bf16",
    ("bfloat16", "16x16x32"): "v_mfma_f32_16x16x32_bf16",
    ("int8", "32x32x32"): "v_mfma_i32_32x32x32_i8",
    ("int8", "16x16x64"): "v_mfma_i32_16x16x64_i8",
}


def mfma_fragment_layout(shape_key):
    """Where the elements of one MFMA issue live in the 64 lanes.

    Every lane holds 16 contiguous bytes of K for one row of A (and one column of B).
    Returns a dict of callables mapping (lane, element) -> matrix coordinates:
      a(lane, e) -> (i, k)   e-th element of the lane's A fragment
      b(lane, e) -> (k, j)
      d(lane, r) -> (i, j)   r-th accumulator register of the lane
    Both are checked on hardware by the parity tests: the direct-to-LDS GEMM kernels issue the
    16x16 shapes (16x16x32 fp16 / bf16, 16x16x64 int8), the register-staged implicit GEMM and
    the patch-staged convolution the 32x32 ones (32x32x16, int8 32x32x32).
    """
    m, n, k = (int(x) for x in shape_key.split("x"))
    per_lane = k * m // 64          # K elements a lane holds (8 halves or 16 int8)
    if m == 32:
        return {
            "a": lambda lane, e: (lane % 32, per_lane * (lane // 32) + e),
            "b": lambda lane, e: (per_lane * (lane // 32) + e, lane % 32),
            "d": lambda lane, r: (8 * (r // 4) + 4 * (lane // 32) + r % 4, lane % 32),
            "acc_regs": 16, "k_per_lane": per_lane,
        }
    return {
        "a": lambda lane, e: (lane % 16, per_lane * (lane // 16) + e),
        "b": lambda lane, e: (per_lane * (lane // 16) + e, lane % 16),
        "d": lambda lane, r: (4 * (lane // 16) + r, lane % 16),
        "acc_regs": 4, "k_per_lane": per_lane,
    }


class MFMABase(ComputeAbstraction):
    """C[i,j] = sum_rk (A(i,rk) * B(rk,j)) widened to the accumulator type.
    (reference semantics: hw_abstraction/cuda/wmma_base.py:439-491)"""
    target = "hip"
    in_dtype = None
    out_dtype = None
    exact_product = False   # int8: operands are widened BEFORE the multiply

    def get_compute_expression(self, input_shapes, output_shape, trans_A=False, trans_B=False, trans_C=False):
        a_shape, b_shape = input_shapes
        m, k_a = (a_shape[1], a_shape[0]) if trans_A else a_shape
        k_b, n = (b_shape[1], b_shape[0]) if trans_B else b_shape
        assert k_a == k_b
        A = te.placeholder(input_shapes[0], name="A", dtype=self.in_dtype)
        B = te.placeholder(input_shapes[1], name="B", dtype=self.in_dtype)
        rk = te.reduce_axis([0, k_a], name="rk")

        def load_a(i):
            return A[rk, i] if trans_A else A[i, rk]

        def load_b(j):
            return B[j, rk] if trans_B else B[rk, j]

        def body(i, j):
            if self.exact_product:
                prod = load_a(i).astype(self.out_dtype) * load_b(j).astype(self.out_dtype)
            else:
                prod = (load_a(i) * load_b(j)).astype(self.out_dtype)
            return te.sum(prod, axis=rk)

        if trans_C:
            C = te.compute([n, m], lambda j, i: body(i, j), name="C")
        else:
            C = te.compute([m, n], lambda i, j: body(i, j), name="C")
        return [A, B], [C]

    def get_intrinsic(self, shape_key):
        return MFMA_INSTRUCTIONS[(self.in_dtype, shape_key)]


@register_abstraction("hip", "mfma_f16_f32::mma")
class MFMAF16F32Mma(MFMABase):
    in_dtype, out_dtype = "float16", "float32"


@register_abstraction("hip", "mfma_bf16_f32::mma")
class MFMABF16F32Mma(MFMABase):
    in_dtype, out_dtype = "bfloat16", "float32"


@register_abstraction("hip", "mfma_i8_i32::mma")
class MFMAI8I32Mma(MFMABase):
    """int8 operands are sign-extended before the multiply (exact int32 products), the
    spelling of python/tvm/auto_tensorize/hw_abstraction/llvm/x86_gemv.py:41-46."""
    in_dtype, out_dtype = "int8", "int32"
    exact_product = True


@register_abstraction("hip", "mfma_i8_i32::mma_wrapped_spelling")
class MFMAI8I32MmaWrappedSpelling(MFMABase):
    """Matches the reference's Tensor Core int8 spelling (a * b).astype("int32")
    (hw_abstraction/cuda/wmma_base.py:439-491).  On the reference's own llvm target that
    multiply wraps to int8 first; the matrix core computes exact products, so results
    differ from the llvm build wherever |a*b| > 127.  Matching it is allowed and flagged."""
    in_dtype, out_dtype = "int8", "int32"
    exact_product = False


class LdsLoad(MemoryAbstraction):
    """LDS -> operand fragment: one ds_read_b128 per lane, rows of eight 16-byte chunks with
    the chunk index XOR-swizzled by the row so that 16 lanes reading 16 rows at one K offset
    hit 16 different bank groups.  Replaces wmma::load_matrix_sync
    (hw_abstraction/cuda/wmma_base.py:176-345)."""
    target = "hip"

    @staticmethod
    def lds_offset(row, chunk):
        return row * 128 + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4)


class GlobalStore(MemoryAbstraction):
    """accumulator -> global memory in the FINAL tensor layout (no tile-major scratch and no
    scatter kernel): register r of lane l goes to row 8*(r/4) + 4*(l/32) + r%4, column l%32
    of the 32x32 tile.  Replaces wmma::store_matrix_sync (wmma_base.py:12-173)."""
    target = "hip"


@register_abstraction("hip", "mfma::add_bias")
class MFMAAddBias(ElementwiseComputeAbstraction):
    """C = A + B.astype(out) on the accumulator registers of a wavefront: the tail a kernel
    fuses into its store.  Replaces nvcuda::wmma::add_bias
    (hw_abstraction/cuda/wmma_bias.py:12-80)."""
    target = "hip"

    def get_compute_expression(self, input_shapes, output_shapes, input_dtypes, output_dtypes, problem_size=None):
        assert len(input_shapes) == 2 and len(output_shapes) == 1
        A = te.placeholder(input_shapes[0], name="A", dtype=input_dtypes[0])
        _, outs = self.get_compute_expression_with_inputs([A], input_shapes, output_shapes, input_dtypes,
                                                          output_dtypes, problem_size)
        return [A, outs[0].op.input_tensors[1]], outs

    def get_compute_expression_with_inputs(self, inputs, input_shapes, output_shapes, input_dtypes,
                                           output_dtypes, problem_size=None):
        (A,) = inputs
        B = te.placeholder(input_shapes[1], name="B", dtype=input_dtypes[1])
        same = input_dtypes[1] == output_dtypes[0]
        C = te.compute(output_shapes[0],
                       lambda *idx: A(*idx) + (B(*idx) if same else B(*idx).astype(output_dtypes[0])), name="C")
        return [A, B], [C]


register_abstraction("hip", "mfma::lds_load")(LdsLoad)
register_abstraction("hip", "mfma::global_store")(GlobalStore)
