"""From a matched TE compute to an operator descriptor of the C ABI.

The reference lowers the mapped compute through TVM's schedule, TIR passes and CUDA code
generator (python/tvm/auto_tensorize/tensorization_phases/schedulers/cuda_v2.py:398-854,
src/target/source/codegen_c.cc:733-772).  Here the kernels exist already; lowering means
recognising which of them a compute is -- GEMM (any of the four operand transpositions),
batched GEMM, NCHW conv2d or NCDHW conv3d with their padding stage -- and reading strides,
dilations, paddings and layouts off the affine index expressions.  A compute that matches
an intrinsic but has no kernel raises NoKernelError; nothing falls back to another device.
"""
from .. import _lib, te


class NoKernelError(RuntimeError):
    pass


class LoweredOp(object):
    """kind: 'gemm' | 'bgemm' | 'conv2d' | 'conv3d'; `inputs` are the two placeholder tensors
    in kernel argument order (row/A operand first for GEMM, activations first for conv);
    `output` the result tensor."""

    def __init__(self, kind, op_code, desc, inputs, output, attrs):
        self.kind = kind
        self.op_code = op_code
        self.desc = desc
        self.inputs = inputs
        self.output = output
        self.attrs = attrs
        self.add_input = None    # tensor D of a fused tail  output = main + D.astype(out), else None
        # {0 or 1: OperandView}: the kernel does not read inputs[k] itself but a tensor gathered
        # from it (stages in front of the operand that no loader folds in), materialised per call
        self.gathers = {}
        # {0 or 1: numpy array}: inputs[k] is computed from its indices alone; the module holds it
        self.constants = {}
        # {0 or 1: EltwiseStage}: inputs[k] is not a placeholder but an element-wise function of
        # placeholders (computed per call by amos_eltwise; a gather may sit on top of it)
        self.computed = {}
        # OperandView (src None) or None: the kernel writes a tensor of the same size in another
        # order and `output` is gathered from it (a stage behind the main op that no epilogue folds in)
        self.out_view = None

    def flops(self):
        a = self.attrs
        if self.kind in ("gemm", "bgemm"):
            return 2.0 * a.get("batch", 1) * a["M"] * a["N"] * a["K"]
        return 2.0 * a["J"] * a["K_out"] * a["K_red"]

    def __str__(self):
        tail = " + %s" % self.add_input.name if self.add_input is not None else ""
        return "%s%s %s" % (self.kind, tail, {k: v for k, v in self.attrs.items()})


def _single_var(form, iters):
    """affine form that is exactly one iteration variable (coefficient 1, constant 0)"""
    if form is None:
        return None
    coef, const = form
    if const != 0 or len(coef) != 1:
        return None
    (v, c), = coef.items()
    if c != 1:
        return None
    for iv in iters:
        if iv.var is v:
            return iv
    return None


class OperandView(object):
    """a tensor every element of which is one element of a placeholder or zero, the source
    index of each dimension depending on that dimension's index alone:
    view[o0, .., on] = src.flat[sum_d tables[d][o_d]] if all tables[d][o_d] >= 0 else 0"""

    def __init__(self, src, shape, tables, dtype):
        self.src, self.shape, self.tables, self.dtype = src, list(shape), tables, dtype


class _NotSeparable(Exception):
    pass


def _eval_int(e, env):
    if isinstance(e, te.IntImm):
        return int(e.value)
    if isinstance(e, te.Var):
        if id(e) not in env:
            raise _NotSeparable("free variable %s" % e.name)
        return env[id(e)]
    if isinstance(e, te.Cast):
        return _eval_int(e.value, env)
    if isinstance(e, te.And):
        return all(_eval_int(t, env) for t in e.terms)
    if isinstance(e, te.Cmp):
        a, b = _eval_int(e.a, env), _eval_int(e.b, env)
        return {"==": a == b, ">=": a >= b, ">": a > b, "<=": a <= b, "<": a < b, "!=": a != b}[e.op]
    if isinstance(e, (te.Add, te.Sub, te.Mul, te.FloorDiv, te.FloorMod)):
        a, b = _eval_int(e.a, env), _eval_int(e.b, env)
        if isinstance(e, te.Add): return a + b
        if isinstance(e, te.Sub): return a - b
        if isinstance(e, te.Mul): return a * b
        if b == 0:
            raise _NotSeparable("division by zero")
        return a // b if isinstance(e, te.FloorDiv) else a % b
    raise _NotSeparable("expression %r" % (e,))


def _vars_in(e, out):
    if isinstance(e, te.Var):
        out[id(e)] = e
    for name in ("a", "b", "value", "cond", "then_value", "else_value"):
        if hasattr(e, name) and isinstance(getattr(e, name), te.Expr):
            _vars_in(getattr(e, name), out)
    for t in getattr(e, "terms", []):
        _vars_in(t, out)
    return out


def _index_tables(indices, variables, extents, src_shape, cond=None):
    """for a load `src[indices]` under `cond`, with every index and every term of the condition a
    function of at most one variable: per variable a list, over its values, of
    {source dimension: index} (None where the condition fails or an index leaves the source);
    indices without a variable come back as a second dictionary"""
    ids = [id(v) for v in variables]
    terms = []
    if cond is not None:
        terms = list(cond.terms) if isinstance(cond, te.And) else [cond]
    term_var = []
    for t in terms:
        vs = [k for k in _vars_in(t, {}) if k in ids]
        if len(vs) > 1:
            raise _NotSeparable("a condition couples two indices")
        term_var.append(ids.index(vs[0]) if vs else None)
    if any(tv is None and not _eval_int(t, {}) for t, tv in zip(terms, term_var)):
        raise _NotSeparable("constant false condition")
    index_var, fixed = [], {}
    for k, idx in enumerate(indices):
        vs = [v for v in _vars_in(idx, {}) if v in ids]
        if len(vs) > 1:
            raise _NotSeparable("an index of %d variables" % len(vs))
        index_var.append(ids.index(vs[0]) if vs else None)
        if not vs:
            fixed[k] = _eval_int(idx, {})
            if not 0 <= fixed[k] < int(src_shape[k]):
                raise _NotSeparable("constant index outside the source")
    stage = []
    for d in range(len(variables)):
        column = []
        for v in range(extents[d]):
            env = {ids[d]: v}
            entry = {}
            if not all(_eval_int(t, env) for t, tv in zip(terms, term_var) if tv == d):
                entry = None
            else:
                for k, idx in enumerate(indices):
                    if index_var[k] == d:
                        x = _eval_int(idx, env)
                        if not 0 <= x < int(src_shape[k]):
                            entry = None
                            break
                        entry[k] = x
            column.append(entry)
        stage.append(column)
    return stage, fixed


class EltwiseStage(object):
    """tensor = f(placeholders at the same index): `inputs` the placeholders, `program` postfix
    steps ("load", k) / ("const", value) / "add" / "sub" / "mul" (ops.Eltwise)"""

    def __init__(self, tensor, inputs, program):
        self.tensor, self.inputs, self.program = tensor, inputs, program


def _eltwise_stage(tensor):
    """EltwiseStage if `tensor` is a compute without reduction whose body is +, -, * over constants
    and loads of placeholders of its own shape and type at exactly its own indices
    (benchmark/amos/mapping_variance_tensorcore.py:12-16), else None"""
    op = tensor.op
    if not isinstance(op, te.ComputeOp) or op.reduce_axis:
        return None
    variables = [iv.var for iv in op.axis]
    shape = [int(e) for e in tensor.shape]
    inputs, program = [], []

    def walk(e):
        if isinstance(e, te.ProducerLoad):
            t = e.tensor
            if not isinstance(t.op, te.PlaceholderOp) or t.dtype != tensor.dtype or \
                    [int(x) for x in t.shape] != shape or len(e.indices) != len(variables) or \
                    any(i is not v for i, v in zip(e.indices, variables)):
                return False
            if all(t is not u for u in inputs):
                inputs.append(t)
            program.append(("load", [k for k, u in enumerate(inputs) if u is t][0]))
            return True
        if isinstance(e, (te.IntImm, te.FloatImm)):
            program.append(("const", float(e.value)))
            return True
        if isinstance(e, te.Cast) and e.dtype == tensor.dtype:
            return walk(e.value)
        if isinstance(e, (te.Add, te.Sub, te.Mul)):
            if not (walk(e.a) and walk(e.b)):
                return False
            program.append({te.Add: "add", te.Sub: "sub", te.Mul: "mul"}[type(e)])
            return True
        return False

    if not walk(op.body[0]) or not inputs or len(inputs) > 4 or len(program) > 16 or \
            sum(1 for p in program if isinstance(p, tuple) and p[0] == "const") > 4:
        return None
    # the register stack of the kernel is four deep
    depth = peak = 0
    for p in program:
        depth += 1 if isinstance(p, tuple) else -1
        peak = max(peak, depth)
    if peak > 4 or tensor.dtype not in ("float16", "bfloat16", "int8"):
        return None
    return EltwiseStage(tensor, inputs, program)


def _operand_view(tensor, head=None, computed_source=False):
    """OperandView of `tensor` (a chain of index-remapping stages over a placeholder); `head`:
    an extra outermost stage (shape, variables, indices into `tensor`), e.g. a load with
    flipped or permuted indices.  With `computed_source` the chain may also end at an element-wise
    function of placeholders (see _eltwise_stage), which then is the view's source."""
    try:
        if head is not None:
            shape, variables, indices = head
            view, fixed = _index_tables(indices, variables, shape, tensor.shape)
        else:
            shape = [int(s) for s in tensor.shape]
            view, fixed = [[{d: o} for o in range(shape[d])] for d in range(len(shape))], {}
        cur = tensor
        while not isinstance(cur.op, te.PlaceholderOp):
            op = cur.op
            if computed_source and _eltwise_stage(cur) is not None and not (
                    isinstance(op.body[0], te.ProducerLoad) or isinstance(op.body[0], te.Select)):
                break      # an element-wise function of placeholders: the view's source is computed per call
            if not isinstance(op, te.ComputeOp) or op.reduce_axis:
                raise _NotSeparable("stage %s reduces" % op.name)
            body, cond = op.body[0], None
            if isinstance(body, te.Select):
                zero = body.else_value
                if not isinstance(zero, (te.IntImm, te.FloatImm)) or zero.value != 0:
                    raise _NotSeparable("a stage fills with something other than zero")
                body, cond = body.then_value, body.cond
            if not isinstance(body, te.ProducerLoad) or body.dtype != cur.dtype:
                raise _NotSeparable("stage %s computes" % op.name)
            stage, sfixed = _index_tables(body.indices, [iv.var for iv in op.axis],
                                          [int(iv.dom.extent) for iv in op.axis], body.tensor.shape, cond)

            def through(entry):
                """coordinates in `cur` -> coordinates in the tensor the stage reads"""
                if entry is None:
                    return None
                out = {}
                for cd, i in entry.items():
                    e = stage[cd][i]
                    if e is None:
                        return None
                    out.update(e)
                return out

            # (coordinates of `cur` fixed by an outer stage go through this stage as well)
            passed = through(fixed)
            if passed is None:
                raise _NotSeparable("a constant index selects a zero")
            view = [[through(e) for e in column] for column in view]
            fixed = dict(sfixed)
            fixed.update(passed)
            cur = body.tensor
        ndim = len(cur.shape)
        owner = {}
        for d, column in enumerate(view):
            for e in column:
                for k in (e or {}):
                    if owner.setdefault(k, d) != d:
                        raise _NotSeparable("a source dimension addressed from two dimensions")
        if sorted(list(owner) + list(fixed)) != list(range(ndim)):
            raise _NotSeparable("a source dimension is not addressed")
    except _NotSeparable as e:
        raise NoKernelError("operand %s is not a per-dimension rearrangement of a placeholder: %s"
                            % (tensor.name, e))
    strides = _row_major_strides([int(s) for s in cur.shape])
    base = sum(i * strides[k] for k, i in fixed.items())
    tables = [[sum(i * strides[k] for k, i in e.items()) if e is not None else -1 for e in column]
              for column in view]
    # the constant part of the address rides on the first dimension's entries
    tables[0] = [t + base if t >= 0 else -1 for t in tables[0]]
    return OperandView(cur, shape, tables, cur.dtype)


def _eval_array(e, env):
    """numpy value of an index-only expression over the index grids in `env`"""
    import numpy as np
    if isinstance(e, (te.IntImm, te.FloatImm)):
        return np.asarray(e.value)
    if isinstance(e, te.Var):
        if id(e) not in env:
            raise _NotSeparable("free variable %s" % e.name)
        return env[id(e)]
    if isinstance(e, te.Cast):
        return _eval_array(e.value, env)
    if isinstance(e, te.And):
        out = np.asarray(True)
        for t in e.terms:
            out = np.logical_and(out, _eval_array(t, env))
        return out
    if isinstance(e, te.Select):
        return np.where(_eval_array(e.cond, env), _eval_array(e.then_value, env), _eval_array(e.else_value, env))
    if isinstance(e, te.Cmp):
        a, b = _eval_array(e.a, env), _eval_array(e.b, env)
        return {"==": a == b, ">=": a >= b, ">": a > b, "<=": a <= b, "<": a < b, "!=": a != b}[e.op]
    if isinstance(e, (te.Add, te.Sub, te.Mul, te.FloorDiv, te.FloorMod)):
        a, b = _eval_array(e.a, env), _eval_array(e.b, env)
        if isinstance(e, te.Add): return a + b
        if isinstance(e, te.Sub): return a - b
        if isinstance(e, te.Mul): return a * b
        return a // b if isinstance(e, te.FloorDiv) else a % b
    raise _NotSeparable("expression %r" % (e,))


def _constant_operand(tensor):
    """host array of a tensor computed from its indices alone (the reference's vector of
    1/n in benchmark/amos/mapping_mean_tensorcore.py:14-16, the triangle of ones in
    mapping_scan_tensorcore.py:9-15), or None"""
    import numpy as np
    op = tensor.op
    if not isinstance(op, te.ComputeOp) or op.reduce_axis or te.collect_loads(op.body[0]):
        return None
    shape = [int(s) for s in tensor.shape]
    grids = np.meshgrid(*[np.arange(n) for n in shape], indexing="ij") if shape else []
    try:
        val = _eval_array(op.body[0], {id(iv.var): g for iv, g in zip(op.axis, grids)})
    except _NotSeparable:
        return None
    if tensor.dtype == "bfloat16":
        raise NoKernelError("constant bfloat16 operands have no host form")
    return np.ascontiguousarray(np.broadcast_to(val, shape).astype(tensor.dtype))


def _strip_cast(e):
    while isinstance(e, te.Cast):
        e = e.value
    return e


def _product_loads(main_op):
    body = main_op.body[0]
    if not isinstance(body, te.Reduce):
        raise NoKernelError("main op is not a sum reduction")
    src = _strip_cast(body.source)
    if not isinstance(src, te.Mul):
        raise NoKernelError("reduction source is not a product")
    l0, l1 = _strip_cast(src.a), _strip_cast(src.b)
    if not (isinstance(l0, te.ProducerLoad) and isinstance(l1, te.ProducerLoad)):
        raise NoKernelError("product operands are not tensor loads")
    return l0, l1


_DT = {"float16": _lib.AMOS_F16, "bfloat16": _lib.AMOS_BF16, "int8": _lib.AMOS_I8,
       "float32": _lib.AMOS_F32, "int32": _lib.AMOS_I32}


def _dtype_pair(l0, l1, out):
    if l0.dtype != l1.dtype or (l0.dtype, out.dtype) not in (("float16", "float32"), ("bfloat16", "float32"),
                                                            ("int8", "int32")):
        raise NoKernelError("no kernel for dtypes %s x %s -> %s" % (l0.dtype, l1.dtype, out.dtype))
    return _DT[l0.dtype], _DT[out.dtype]


def _lower_gemm(main_op, l0, l1, iters, forms0, forms1):
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    if len(reduce_) != 1 or len(spatial) not in (2, 3):
        return None
    k = reduce_[0]
    v0 = [_single_var(f, iters) for f in forms0]
    v1 = [_single_var(f, iters) for f in forms1]
    if any(v is None for v in v0 + v1) or len(v0) != len(spatial) or len(v1) != len(spatial):
        return None
    batch = spatial[0] if len(spatial) == 3 else None
    x, y = spatial[-2], spatial[-1]
    if batch is not None and (v0[0] is not batch or v1[0] is not batch):
        return None
    d0, d1 = v0[-2:], v1[-2:]

    def has(d, iv):
        return any(e is iv for e in d)

    if has(d0, x) and has(d1, y) and not has(d0, y) and not has(d1, x):
        la, lb, da, db = l0, l1, d0, d1
    elif has(d1, x) and has(d0, y) and not has(d1, y) and not has(d0, x):
        la, lb, da, db = l1, l0, d1, d0
    else:
        return None
    if not (has(da, k) and has(db, k)):
        return None
    # an operand that is computed: a constant (a function of its indices), or a per-dimension
    # rearrangement of a placeholder that is materialised in front of the kernel
    sources, gathers, constants, computed = [la.tensor, lb.tensor], {}, {}, {}
    for pos, ld in enumerate((la, lb)):
        if isinstance(ld.tensor.op, te.PlaceholderOp):
            continue
        const = _constant_operand(ld.tensor)
        if const is not None:
            constants[pos] = const
        else:
            gathers[pos] = _operand_view(ld.tensor, computed_source=True)
            sources[pos] = gathers[pos].src
            if not isinstance(sources[pos].op, te.PlaceholderOp):
                computed[pos] = _eltwise_stage(sources[pos])
    trans_a = 0 if da[0] is x else 1          # [x, k] row-major A, [k, x] transposed
    trans_b = 0 if db[0] is k else 1          # [k, y] row-major B, [y, k] column-major B
    M, N, K = int(x.dom.extent), int(y.dom.extent), int(k.dom.extent)
    ind, outd = _dtype_pair(la, lb, main_op.output(0))
    g = _lib.GemmDesc()
    g.M, g.N, g.K, g.in_dtype, g.out_dtype, g.trans_a, g.trans_b = M, N, K, ind, outd, trans_a, trans_b
    g.lda, g.ldb, g.ldc = (M if trans_a else K), (K if trans_b else N), N
    attrs = dict(M=M, N=N, K=K, trans_a=trans_a, trans_b=trans_b, dtype=la.dtype)
    if batch is None:
        low = LoweredOp("gemm", _lib.AMOS_OP_GEMM, g, sources, main_op.output(0), attrs)
    else:
        b = _lib.BGemmDesc()
        b.batch = int(batch.dom.extent)
        b.g = g
        b.stride_a, b.stride_b, b.stride_c = M * K, K * N, M * N
        attrs["batch"] = b.batch
        low = LoweredOp("bgemm", _lib.AMOS_OP_BGEMM, b, sources, main_op.output(0), attrs)
    low.gathers, low.constants, low.computed = gathers, constants, computed
    return low


def _row_major_strides(shape):
    strides, acc = [], 1
    for ext in reversed([int(x) for x in shape]):
        strides.append(acc)
        acc *= ext
    return list(reversed(strides))


def _flat_address(load, variables):
    """Element offset of a tensor load inside the PLACEHOLDER it ultimately reads, as an affine
    form ({Var: coefficient}, constant) of `variables`.  Pure view stages in between -- computes
    without a reduction whose body is one load with affine indices, the reshapes of
    benchmark/amos/mapping_batchedfc_tensorcore.py:14-22 -- are substituted away.  None when
    the chain is not affine or changes values."""
    forms = [te.affine_form(i, variables) for i in load.indices]
    if any(f is None for f in forms):
        return None
    op = load.tensor.op
    if isinstance(op, te.PlaceholderOp):
        coef, const = {}, 0
        for f, stride in zip(forms, _row_major_strides(load.tensor.shape)):
            for v, c in f[0].items():
                coef[v] = coef.get(v, 0) + c * stride
            const += f[1] * stride
        return load.tensor, {v: c for v, c in coef.items() if c != 0}, const
    if not isinstance(op, te.ComputeOp) or op.reduce_axis:
        return None
    inner = op.body[0]
    if isinstance(inner, te.Cast) and inner.dtype == inner.value.dtype:
        inner = inner.value
    if not isinstance(inner, te.ProducerLoad) or inner.dtype != load.dtype:
        return None
    view_vars = [iv.var for iv in op.axis]
    res = _flat_address(inner, view_vars)
    if res is None:
        return None
    src, icoef, iconst = res
    coef, const = {}, iconst
    for vv, f in zip(view_vars, forms):       # substitute view variable := the load's index form
        c = icoef.get(vv, 0)
        if c == 0:
            continue
        for v, cc in f[0].items():
            coef[v] = coef.get(v, 0) + c * cc
        const += c * f[1]
    return src, {v: c for v, c in coef.items() if c != 0}, const


def _lower_strided_gemm(main_op, l0, l1):
    """GEMM, batched GEMM and their strided relatives (GEMV, batched FC over channel groups,
    operands read through reshaping stages) from the flat addresses of the two loads: a spatial
    iteration variable in one operand only is M or N, in both it is the batch; leading
    dimensions and batch strides are the coefficients.  (reference computes:
    benchmark/amos/mapping_gemm_tensorcore.py:7-15, mapping_gemv_tensorcore.py:7-16,
    mapping_batchedfc_tensorcore.py:7-37)"""
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    if len(reduce_) != 1:
        return None
    variables = [iv.var for iv in spatial + reduce_]
    r0, r1 = _flat_address(l0, variables), _flat_address(l1, variables)
    if r0 is None or r1 is None or r0[2] != 0 or r1[2] != 0:
        return None
    k = reduce_[0]
    if k.var not in r0[1] or k.var not in r1[1]:
        return None
    live = [iv for iv in spatial if int(iv.dom.extent) > 1]
    in0 = [iv for iv in live if iv.var in r0[1]]
    in1 = [iv for iv in live if iv.var in r1[1]]
    batch = [iv for iv in in0 if any(iv is j for j in in1)]
    only0 = [iv for iv in in0 if not any(iv is j for j in batch)]
    only1 = [iv for iv in in1 if not any(iv is j for j in batch)]
    if len(batch) > 1 or len(only0) > 1 or len(only1) > 1 or len(batch) + len(only0) + len(only1) != len(live):
        return None
    out_strides = dict(zip([iv.var for iv in spatial], _row_major_strides(main_op.output(0).shape)))

    def roles(ra, rb, m_iv, n_iv):
        """A-side / B-side description with (m_iv from ra, n_iv from rb), or None"""
        K = int(k.dom.extent)
        M = int(m_iv.dom.extent) if m_iv is not None else 1
        N = int(n_iv.dom.extent) if n_iv is not None else 1
        a_m = ra[1].get(m_iv.var, 0) if m_iv is not None else 0
        a_k = ra[1][k.var]
        b_n = rb[1].get(n_iv.var, 0) if n_iv is not None else 0
        b_k = rb[1][k.var]
        if a_k == 1 and (M == 1 or a_m >= K):
            trans_a, lda = 0, (a_m if M > 1 else K)
        elif (a_m == 1 or M == 1) and a_k >= M:
            trans_a, lda = 1, a_k
        else:
            return None
        if b_k == 1 and (N == 1 or b_n >= K):
            trans_b, ldb = 1, (b_n if N > 1 else K)
        elif (b_n == 1 or N == 1) and b_k >= N:
            trans_b, ldb = 0, b_k
        else:
            return None
        c_m = out_strides[m_iv.var] if m_iv is not None else N
        c_n = out_strides[n_iv.var] if n_iv is not None else 1
        if (N > 1 and c_n != 1) or (M > 1 and c_m < N):
            return None
        return dict(M=M, N=N, K=K, trans_a=trans_a, trans_b=trans_b, lda=lda, ldb=ldb, ldc=c_m if M > 1 else N)

    m_iv = only0[0] if only0 else None
    n_iv = only1[0] if only1 else None
    la, lb, ra, rb = l0, l1, r0, r1
    g = roles(ra, rb, m_iv, n_iv)
    if g is None:       # the other operand supplies the output rows
        la, lb, ra, rb, m_iv, n_iv = l1, l0, r1, r0, n_iv, m_iv
        g = roles(ra, rb, m_iv, n_iv)
    if g is None:
        return None
    ind, outd = _dtype_pair(la, lb, main_op.output(0))
    d = _lib.GemmDesc()
    d.M, d.N, d.K, d.in_dtype, d.out_dtype = g["M"], g["N"], g["K"], ind, outd
    d.trans_a, d.trans_b, d.lda, d.ldb, d.ldc = g["trans_a"], g["trans_b"], g["lda"], g["ldb"], g["ldc"]
    attrs = dict(M=g["M"], N=g["N"], K=g["K"], trans_a=g["trans_a"], trans_b=g["trans_b"], dtype=la.dtype,
                 lda=g["lda"], ldb=g["ldb"], ldc=g["ldc"])
    if not batch:
        return LoweredOp("gemm", _lib.AMOS_OP_GEMM, d, [ra[0], rb[0]], main_op.output(0), attrs)
    b_iv = batch[0]
    bd = _lib.BGemmDesc()
    bd.batch = int(b_iv.dom.extent)
    bd.g = d
    bd.stride_a, bd.stride_b, bd.stride_c = ra[1][b_iv.var], rb[1][b_iv.var], out_strides[b_iv.var]
    attrs.update(batch=bd.batch, stride_a=bd.stride_a, stride_b=bd.stride_b, stride_c=bd.stride_c)
    return LoweredOp("bgemm", _lib.AMOS_OP_BGEMM, bd, [ra[0], rb[0]], main_op.output(0), attrs)


def _pad_stage(tensor, spatial_dims=None):
    """tensor made by the padding compute -> (source placeholder, pads per spatial dim);
    spatial_dims: which dimensions may be padded (default: all but the first two)"""
    op = tensor.op
    if spatial_dims is None:
        spatial_dims = list(range(2, len(tensor.shape)))
    if isinstance(op, te.PlaceholderOp):
        return tensor, [0] * len(spatial_dims)
    if not isinstance(op, te.ComputeOp) or op.reduce_axis:
        raise NoKernelError("activation operand is neither a placeholder nor a padding stage")
    body = op.body[0]
    if not isinstance(body, te.Select) or not isinstance(_strip_cast(body.then_value), te.ProducerLoad):
        raise NoKernelError("unrecognised stage %s in front of the convolution" % op.name)
    zero = body.else_value
    if not isinstance(zero, (te.IntImm, te.FloatImm)) or zero.value != 0:
        raise NoKernelError("padding value is not zero")
    load = _strip_cast(body.then_value)
    src = load.tensor
    if not isinstance(src.op, te.PlaceholderOp):
        raise NoKernelError("padding stage does not read a placeholder")
    variables = [iv.var for iv in op.axis]
    pads = {}
    for d, idx in enumerate(load.indices):
        form = te.affine_form(idx, variables)
        if form is None or len(form[0]) != 1 or list(form[0].items())[0] != (variables[d], 1):
            raise NoKernelError("padding stage permutes or scales indices")
        pad = -form[1]
        if d not in spatial_dims:
            if pad != 0:
                raise NoKernelError("padding on the batch or channel dimension")
        else:
            if pad < 0 or int(op.output(0).shape[d]) != int(src.shape[d]) + 2 * pad:
                raise NoKernelError("padding stage is not symmetric zero padding")
            pads[d] = pad
    return src, [pads[d] for d in spatial_dims]


# where batch / channel / spatial dimensions sit in the three tensors of a convolution
# (reference: the three layouts of benchmark/amos/mapping_conv2d_tensorcore.py:7-104)
def _conv_templates(nsp):
    sp = list(range(nsp))
    return [
        # name, x: (n, c, spatial), w: (k, c, window), out: (n, k, spatial)
        ("nchw", (0, 1, [2 + d for d in sp]), (0, 1, [2 + d for d in sp]), (0, 1, [2 + d for d in sp])),
        ("nhwc", (0, nsp + 1, [1 + d for d in sp]), (nsp + 1, nsp, sp), (0, nsp + 1, [1 + d for d in sp])),
        ("hwnc", (nsp, nsp + 1, sp), (nsp + 1, nsp, sp), (nsp, nsp + 1, sp)),
    ]


def _lower_conv(main_op, l0, l1, iters, forms0, forms1):
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    nsp = len(spatial) - 2                     # 1, 2 or 3 spatial output dims
    if nsp not in (1, 2, 3) or len(reduce_) != nsp + 1:
        return None

    def try_roles(template, lx, fx, lw, fw):
        _, (xn, xc, xsp), (wk, wc, wsp), (on, ok, osp) = template
        if len(fx) != nsp + 2 or len(fw) != nsp + 2:
            return None
        n_iv, k_iv, out_sp = spatial[on], spatial[ok], [spatial[d] for d in osp]
        # the activations say which reduce axis is the channel and which belongs to which
        # spatial dimension
        rc = _single_var(fx[xc], iters)
        if _single_var(fx[xn], iters) is not n_iv or rc is None or all(rc is not r for r in reduce_):
            return None
        strides, dils, red_sp = [], [], []
        for d in range(nsp):
            f = fx[xsp[d]]
            if f is None:
                return None
            coef, const = f
            rv = [iv for iv in reduce_ if iv.var in coef]
            if const != 0 or len(rv) > 1 or set(coef.keys()) - {out_sp[d].var} - {iv.var for iv in rv}:
                return None
            # (a 1-wide window has a reduce axis of extent 1 that may be folded away)
            red_sp.append(rv[0] if rv else None)
            strides.append(int(coef.get(out_sp[d].var, 1)))
            dils.append(int(coef[rv[0].var]) if rv else 1)
            if strides[-1] < 1 or dils[-1] < 1:
                return None
        # the weights: laid out as the template says, or any per-dimension rearrangement of the
        # same axes (flipped windows, swapped channel dimensions: gathered into the template's order)
        wv = [_single_var(f, iters) for f in fw]
        canonical = wv[wk] is k_iv and wv[wc] is rc and all(
            wv[wsp[d]] is not None and (red_sp[d] is None or wv[wsp[d]] is red_sp[d]) for d in range(nsp))
        if canonical:
            red_sp = [wv[wsp[d]] for d in range(nsp)]
        else:
            per_dim = []
            for idx in lw.indices:
                vs = [iv for iv in iters if id(iv.var) in _vars_in(idx, {})]
                if len(vs) != 1:
                    return None
                per_dim.append(vs[0])
            left = [r for r in reduce_ if r is not rc and all(r is not q for q in red_sp)]
            red_sp = [q if q is not None else left.pop(0) for q in red_sp if q is not None or left]
            if len(red_sp) != nsp or sorted(id(v) for v in per_dim) != sorted(id(v) for v in [k_iv, rc] + red_sp):
                return None
        if sorted(id(r) for r in [rc] + red_sp) != sorted(id(r) for r in reduce_):
            return None
        return strides, dils, rc, red_sp, out_sp, k_iv, canonical

    found = None
    for template in _conv_templates(nsp):
        for lx, fx, lw, fw in ((l0, forms0, l1, forms1), (l1, forms1, l0, forms0)):
            roles = try_roles(template, lx, fx, lw, fw)
            if roles is not None:
                found = (template, lx, lw, roles)
                break
        if found:
            break
    if found is None:
        return None
    template, lx, lw, (strides, dils, rc, red_sp, out_sp, k_iv, canonical) = found
    layout, (xn, xc, xsp), (wk, wc, wsp), _ = template
    gathers = {}
    try:
        src, pads = _pad_stage(lx.tensor, xsp)
        xs_mem = [int(s) for s in src.shape]
    except NoKernelError:
        # stages other than one symmetric zero padding (the zero expansion and one-sided padding
        # of a transposed convolution ...): materialised, the kernel then reads a dense tensor
        view = _operand_view(lx.tensor)
        src, pads, xs_mem = view.src, [0] * nsp, list(view.shape)
        gathers[0] = view
    if canonical and isinstance(lw.tensor.op, te.PlaceholderOp):
        wt, ws_mem = lw.tensor, [int(s) for s in lw.tensor.shape]
    else:
        head = None
        if not canonical:
            order = [None] * (nsp + 2)
            order[wk], order[wc] = k_iv, rc
            for d in range(nsp):
                order[wsp[d]] = red_sp[d]
            head = ([int(iv.dom.extent) for iv in order], [iv.var for iv in order], lw.indices)
        view = _operand_view(lw.tensor, head)
        wt, ws_mem = view.src, list(view.shape)
        gathers[1] = view
    # logical extents: N, C, spatial...; K, C, window...
    xs = [xs_mem[xn], xs_mem[xc]] + [xs_mem[d] for d in xsp]
    ws = [ws_mem[wk], ws_mem[wc]] + [ws_mem[d] for d in wsp]
    for d in range(nsp):
        if int(red_sp[d].dom.extent) != ws[2 + d]:
            raise NoKernelError("reduce extent %d differs from the kernel window %d"
                                % (int(red_sp[d].dom.extent), ws[2 + d]))
        want = (xs[2 + d] + 2 * pads[d] - ((ws[2 + d] - 1) * dils[d] + 1)) // strides[d] + 1
        if int(out_sp[d].dom.extent) != want:
            raise NoKernelError("output extent %d is not what stride / padding / dilation give (%d)"
                                % (int(out_sp[d].dom.extent), want))
    if xs[1] != ws[1] or int(rc.dom.extent) != xs[1]:
        raise NoKernelError("grouped convolution has no kernel")
    ind, outd = _dtype_pair(lx, lw, main_op.output(0))
    c = _lib.ConvDesc()
    if nsp == 1:      # conv1d (benchmark/amos/mapping_conv1d_tensorcore.py:25-42) = conv2d with H = R = 1
        xs5, ws5 = [xs[0], xs[1], 1, 1, xs[2]], [ws[0], ws[1], 1, 1, ws[2]]
        st, pd, dl = [1, 1] + strides, [0, 0] + pads, [1, 1] + dils
    elif nsp == 2:
        xs5, ws5 = [xs[0], xs[1], 1, xs[2], xs[3]], [ws[0], ws[1], 1, ws[2], ws[3]]
        st, pd, dl = [1] + strides, [0] + pads, [1] + dils
    else:
        xs5, ws5, st, pd, dl = xs, ws, strides, pads, dils
    c.N, c.C, c.D, c.H, c.W = xs5
    c.K, _, c.T, c.R, c.S = ws5
    c.stride_d, c.stride_h, c.stride_w = st
    c.pad_d, c.pad_h, c.pad_w = pd
    c.dil_d, c.dil_h, c.dil_w = dl
    c.in_dtype, c.out_dtype = ind, outd
    c.layout = _lib.LAYOUT_CODE[layout]
    J = _numel(main_op.output(0).shape) // ws[0]
    attrs = dict(x_shape=xs, w_shape=ws, stride=strides, pad=pads, dil=dils, dtype=lx.dtype, J=J,
                 K_out=ws[0], K_red=ws[1] * (ws5[2] * ws5[3] * ws5[4]), layout=layout)
    kind, code = ("conv2d", _lib.AMOS_OP_CONV2D) if nsp <= 2 else ("conv3d", _lib.AMOS_OP_CONV3D)
    low = LoweredOp(kind, code, c, [src, wt], main_op.output(0), attrs)
    low.gathers = gathers
    return low


def remap_conv2d_rows(low, rows):
    """The same convolution with only the loops in `rows` (a subset of 'n', 'p', 'q' that holds 'n')
    fused into the rows of the implicit GEMM, the other output loops being time loops: every value
    of such a loop is a convolution of its own, with its own copy of the input rows / columns it
    reads (no reuse of the halo between neighbouring outputs along that loop), all of them batched
    into one launch.  The reference reaches the same loop structure by fusing only the mapped
    loops into the intrinsic's axis (tensorization_phases/compute_transform.py:343-499).

      rows n,q (p a time loop): image n holds, for every output row p, its own R input rows, one
                                block under the other; window R x S, stride R along H
      rows n,p (q a time loop): the same with H and W swapped (the copied axis is the image's H):
                                per output column q its own S input columns; window S x R
      rows n (p, q time loops): one image of P blocks of R rows and N*Q blocks of S columns;
                                window R x S, strides R and S

    `rows` may end in "+s" or "+r": that window loop joins the channels in the reduction of the
    implicit GEMM (rk <- {rc, rs} or {rc, rr}) while the other window loop stays a time loop.  The
    axis of the folded loop is copied tap by tap as above -- per output column q its S input
    columns, side by side -- and the S copies of a column then ARE S * C channels of an image of
    width Q (the same memory, NHWC), convolved with a window R x 1; "+r" is the same with H and W
    swapped.  The output loop of the folded axis is a row loop of necessity (q with "+s", p with
    "+r").

    The copies are dimension-separable gathers (zero padding along the copied axis included) into
    NHWC images; the weights are gathered into the window-major layout that goes with it and the
    result is gathered back to NKPQ."""
    rows, _, fold = rows.partition("+")
    rows = "".join(sorted(rows))
    if fold:
        return _remap_conv2d_fold(low, rows, fold)
    if rows == "npq":
        return low
    if low.kind != "conv2d" or low.attrs.get("layout", "nchw") != "nchw" or low.gathers or low.out_view is not None \
            or low.constants or low.computed or len(low.attrs["x_shape"]) != 4 or rows not in ("nq", "np", "n"):
        raise NoKernelError("no kernel for this convolution with rows %s" % rows)
    N, C, H, W = low.attrs["x_shape"]
    K, _, R, S = low.attrs["w_shape"]
    (sh, sw), (ph, pw), (dh, dw) = low.attrs["stride"], low.attrs["pad"], low.attrs["dil"]
    P = (H + 2 * ph - ((R - 1) * dh + 1)) // sh + 1
    Q = (W + 2 * pw - ((S - 1) * dw + 1)) // sw + 1
    src, wt = low.inputs
    hw = H * W
    # source offsets of the copied axes: (output index, tap) -> input row / column, -1 in the padding
    rows_of = [(p * sh - ph + r * dh) * W if 0 <= p * sh - ph + r * dh < H else -1 for p in range(P) for r in range(R)]
    cols_of = [q * sw - pw + s * dw if 0 <= q * sw - pw + s * dw < W else -1 for q in range(Q) for s in range(S)]
    n_tab, c_tab = [n * C * hw for n in range(N)], [c * hw for c in range(C)]
    c = _lib.ConvDesc()
    c.C, c.K, c.D, c.T = C, K, 1, 1
    c.stride_d, c.pad_d, c.dil_d = 1, 0, 1
    c.stride_h, c.pad_h, c.dil_h = 1, 0, 1
    c.in_dtype, c.out_dtype = low.desc.in_dtype, low.desc.out_dtype
    c.layout = _lib.LAYOUT_CODE["nhwc"]
    krs = C * R * S
    if rows == "nq":
        x_view = OperandView(src, [N, P * R, W, C], [n_tab, rows_of, list(range(W)), c_tab], src.dtype)
        c.N, c.H, c.W, c.R, c.S = N, P * R, W, R, S
        c.stride_h = R
        c.stride_w, c.pad_w, c.dil_w = sw, pw, dw
        w_view = OperandView(wt, [R, S, C, K], [[r * S for r in range(R)], list(range(S)), [cc * R * S for cc in range(C)],
                                                [k * krs for k in range(K)]], wt.dtype)
        o_tabs = [[n * P * Q * K for n in range(N)], list(range(K)), [p * Q * K for p in range(P)], [q * K for q in range(Q)]]
    elif rows == "np":
        x_view = OperandView(src, [N, Q * S, H, C], [n_tab, cols_of, [h * W for h in range(H)], c_tab], src.dtype)
        c.N, c.H, c.W, c.R, c.S = N, Q * S, H, S, R
        c.stride_h = S
        c.stride_w, c.pad_w, c.dil_w = sh, ph, dh
        w_view = OperandView(wt, [S, R, C, K], [list(range(S)), [r * S for r in range(R)], [cc * R * S for cc in range(C)],
                                                [k * krs for k in range(K)]], wt.dtype)
        o_tabs = [[n * Q * P * K for n in range(N)], list(range(K)), [p * K for p in range(P)], [q * P * K for q in range(Q)]]
    else:
        x_view = OperandView(src, [P * R, N, Q * S, C], [rows_of, n_tab, cols_of, c_tab], src.dtype)
        c.N, c.H, c.W, c.R, c.S = 1, P * R, N * Q * S, R, S
        c.stride_h = R
        c.stride_w, c.pad_w, c.dil_w = S, 0, 1
        w_view = OperandView(wt, [R, S, C, K], [[r * S for r in range(R)], list(range(S)), [cc * R * S for cc in range(C)],
                                                [k * krs for k in range(K)]], wt.dtype)
        o_tabs = [[n * Q * K for n in range(N)], list(range(K)), [p * N * Q * K for p in range(P)], [q * K for q in range(Q)]]
    attrs = dict(low.attrs, layout="nhwc", rows=rows)
    out = LoweredOp("conv2d", low.op_code, c, [src, wt], low.output, attrs)
    out.add_input = low.add_input
    out.gathers = {0: x_view, 1: w_view}
    out.out_view = OperandView(None, [N, K, P, Q], o_tabs, low.output.dtype)
    return out


def _remap_conv2d_fold(low, rows, fold):
    """remap_conv2d_rows with one window loop folded into the channels: fold 's' (rows 'npq' or
    'nq') or 'r' (rows 'npq' or 'np')"""
    ok_rows = {"s": ("npq", "nq"), "r": ("npq", "np")}.get(fold, ())
    if low.kind != "conv2d" or low.attrs.get("layout", "nchw") != "nchw" or low.gathers or low.out_view is not None \
            or low.constants or low.computed or len(low.attrs["x_shape"]) != 4 or rows not in ok_rows:
        raise NoKernelError("no kernel for this convolution with rows %s and window loop %s in the reduction" % (rows, fold))
    N, C, H, W = low.attrs["x_shape"]
    K, _, R, S = low.attrs["w_shape"]
    (sh, sw), (ph, pw), (dh, dw) = low.attrs["stride"], low.attrs["pad"], low.attrs["dil"]
    P = (H + 2 * ph - ((R - 1) * dh + 1)) // sh + 1
    Q = (W + 2 * pw - ((S - 1) * dw + 1)) // sw + 1
    src, wt = low.inputs
    hw, krs = H * W, C * R * S
    rows_of = [(p * sh - ph + r * dh) * W if 0 <= p * sh - ph + r * dh < H else -1 for p in range(P) for r in range(R)]
    cols_of = [q * sw - pw + s * dw if 0 <= q * sw - pw + s * dw < W else -1 for q in range(Q) for s in range(S)]
    n_tab, c_tab = [n * C * hw for n in range(N)], [c * hw for c in range(C)]
    c = _lib.ConvDesc()
    c.N, c.K, c.D, c.T = N, K, 1, 1
    c.stride_d, c.pad_d, c.dil_d = 1, 0, 1
    c.in_dtype, c.out_dtype = low.desc.in_dtype, low.desc.out_dtype
    c.layout = _lib.LAYOUT_CODE["nhwc"]
    c.S, c.stride_w, c.pad_w, c.dil_w = 1, 1, 0, 1     # the folded axis: one output per S * C (R * C) channels
    if fold == "s":
        # image [N][H or P*R][Q*S][C] = [N][.][Q][S*C]; window R x 1
        if "p" in rows:
            a_tab, c.H, c.stride_h, c.pad_h, c.dil_h = [h * W for h in range(H)], H, sh, ph, dh
        else:
            a_tab, c.H, c.stride_h, c.pad_h, c.dil_h = rows_of, P * R, R, 0, 1
        x_view = OperandView(src, [N, c.H, Q * S, C], [n_tab, a_tab, cols_of, c_tab], src.dtype)
        c.W, c.C, c.R = Q, S * C, R
        w_view = OperandView(wt, [R, S, C, K], [[r * S for r in range(R)], list(range(S)), [cc * R * S for cc in range(C)],
                                                [k * krs for k in range(K)]], wt.dtype)
        o_tabs = [[n * P * Q * K for n in range(N)], list(range(K)), [p * Q * K for p in range(P)], [q * K for q in range(Q)]]
    else:
        # transposed image [N][W or Q*S][P*R][C] = [N][.][P][R*C]; window S x 1
        if "q" in rows:
            a_tab, c.H, c.stride_h, c.pad_h, c.dil_h = list(range(W)), W, sw, pw, dw
        else:
            a_tab, c.H, c.stride_h, c.pad_h, c.dil_h = cols_of, Q * S, S, 0, 1
        x_view = OperandView(src, [N, c.H, P * R, C], [n_tab, a_tab, rows_of, c_tab], src.dtype)
        c.W, c.C, c.R = P, R * C, S
        w_view = OperandView(wt, [S, R, C, K], [list(range(S)), [r * S for r in range(R)], [cc * R * S for cc in range(C)],
                                                [k * krs for k in range(K)]], wt.dtype)
        o_tabs = [[n * Q * P * K for n in range(N)], list(range(K)), [p * K for p in range(P)], [q * P * K for q in range(Q)]]
    attrs = dict(low.attrs, layout="nhwc", rows=rows + "+" + fold)
    out = LoweredOp("conv2d", low.op_code, c, [src, wt], low.output, attrs)
    out.add_input = low.add_input
    out.gathers = {0: x_view, 1: w_view}
    out.out_view = OperandView(None, [N, K, P, Q], o_tabs, low.output.dtype)
    return out


def _numel(shape):
    n = 1
    for e in shape:
        n *= int(e)
    return n


def _dense_output(low):
    """the kernel writes the main op's tensor contiguously (no padding between rows / batches)"""
    if low.kind == "gemm":
        return low.desc.ldc == low.desc.N
    if low.kind == "bgemm":
        return low.desc.g.ldc == low.desc.g.N and low.desc.stride_c == low.desc.g.M * low.desc.g.N
    return True


def _flat_address_of_compute(load, producer_op, variables):
    """offset of a load of `producer_op`'s (row-major) result, affine in `variables`.  An index
    pair (v // c, v % c) whose strides are (c*s, s) counts as v*s: the split of one axis in two
    that mapping_groupedconv2d_tensorcore.py:53-57 undoes behind its main op."""
    if load.tensor.op is not producer_op:
        return None
    coef, const, div, mod = {}, 0, {}, {}
    for idx, stride in zip(load.indices, _row_major_strides(load.tensor.shape)):
        e = _strip_cast(idx)
        if isinstance(e, (te.FloorDiv, te.FloorMod)) and isinstance(e.a, te.Var) and isinstance(e.b, te.IntImm) \
                and any(e.a is v for v in variables):
            bucket = div if isinstance(e, te.FloorDiv) else mod
            key = (e.a, int(e.b.value))
            bucket[key] = bucket.get(key, 0) + stride
            continue
        f = te.affine_form(idx, variables)
        if f is None:
            return None
        for v, c in f[0].items():
            coef[v] = coef.get(v, 0) + c * stride
        const += f[1] * stride
    if set(div) != set(mod):
        return None
    for (v, c), s_mod in mod.items():
        if div[(v, c)] != c * s_mod:
            return None
        coef[v] = coef.get(v, 0) + s_mod
    return {v: c for v, c in coef.items() if c != 0}, const


def _fuse_tail(low, main_op, target_dag):
    """The element-wise stage behind the main op, if any, becomes the kernel's fused tail.
    The reference keeps such stages in IntrinMatchResult.elem_op_map and maps them with the
    main op (intrin_match.py:24-42, tests/python/auto_tensorize/test_compute_transform_gemm.py:7-23,
    "E = C + D"); the kernels here add one operand of the output's shape on the accumulators."""
    readers = [op for op in target_dag.op_lst if any(t.op is main_op for t in op.input_tensors)]
    if not readers:
        return low
    if len(readers) > 1:
        raise NoKernelError("the main op feeds %d stages; one element-wise tail can be fused" % len(readers))
    tail = readers[0]
    if any(any(t.op is tail for t in op.input_tensors) for op in target_dag.op_lst):
        raise NoKernelError("a chain of stages behind the main op has no fused kernel")
    body = tail.body[0] if not tail.reduce_axis else None
    if isinstance(_strip_cast(body), te.ProducerLoad) and _strip_cast(body).dtype == low.output.dtype:
        # a reshape of the result (mapping_gemv_tensorcore.py:15, D[i] = C[i, 0]): same memory
        variables = [iv.var for iv in tail.axis]
        res = _flat_address_of_compute(_strip_cast(body), main_op, variables)
        want = dict(zip(variables, _row_major_strides(tail.output(0).shape)))
        want = {v: c for v, c in want.items() if int([iv for iv in tail.axis if iv.var is v][0].dom.extent) > 1}
        if res is not None and res[1] == 0 and {v: c for v, c in res[0].items() if v in want} == want and \
                _numel(tail.output(0).shape) == _numel(main_op.output(0).shape) and _dense_output(low):
            low.output = tail.output(0)
            return low
        raise NoKernelError("stage %s behind the main op is neither a reshape nor an addition" % tail.name)
    if not isinstance(body, te.Add):
        raise NoKernelError("stage %s behind the main op is not an element-wise addition" % tail.name)
    loads = [_strip_cast(body.a), _strip_cast(body.b)]
    if not all(isinstance(l, te.ProducerLoad) for l in loads):
        raise NoKernelError("stage %s does not add two tensor elements" % tail.name)
    main_load = [l for l in loads if l.tensor.op is main_op]
    other = [l for l in loads if l.tensor.op is not main_op]
    if len(main_load) != 1 or len(other) != 1 or not isinstance(other[0].tensor.op, te.PlaceholderOp):
        raise NoKernelError("stage %s must add the main op's result and a placeholder" % tail.name)
    variables = [iv.var for iv in tail.axis]
    for l in loads:
        if len(l.indices) != len(variables) or any(i is not v for i, v in zip(l.indices, variables)):
            raise NoKernelError("stage %s permutes or offsets indices" % tail.name)
    d = other[0].tensor
    out = tail.output(0)
    if [int(x) for x in d.shape] != [int(x) for x in out.shape] or out.dtype != low.output.dtype:
        raise NoKernelError("the added tensor must have the output's shape and the sum its type")
    ok = ("int32",) if out.dtype == "int32" else ("float32", "float16", "bfloat16")
    if d.dtype not in ok:
        raise NoKernelError("cannot add a %s tensor to a %s result" % (d.dtype, out.dtype))
    low.add_input = d
    low.output = out
    return low


def _resolve_dims(load, variables):
    """(tensor, per-dimension affine index forms in `variables`) of the first tensor behind `load`
    that is not a pure view stage; None if an index is not affine"""
    forms = [te.affine_form(i, variables) for i in load.indices]
    if any(f is None for f in forms):
        return None
    op = load.tensor.op
    if isinstance(op, te.ComputeOp) and not op.reduce_axis:
        inner = op.body[0]
        if isinstance(inner, te.Cast) and inner.dtype == inner.value.dtype:
            inner = inner.value
        if isinstance(inner, te.ProducerLoad) and inner.dtype == load.dtype:
            view_vars = [iv.var for iv in op.axis]
            res = _resolve_dims(inner, view_vars)
            if res is None:
                return None
            tensor, inner_forms = res
            out = []
            for icoef, iconst in inner_forms:       # substitute view variable := the load's index form
                coef, const = {}, iconst
                for vv, f in zip(view_vars, forms):
                    c = icoef.get(vv, 0)
                    for v, cc in f[0].items():
                        coef[v] = coef.get(v, 0) + c * cc
                    const += c * f[1]
                out.append(({v: c for v, c in coef.items() if c != 0}, const))
            return tensor, out
    return load.tensor, forms


def _lower_grouped_conv(main_op, l0, l1):
    """Grouped and depthwise convolution as the reference spells them
    (benchmark/amos/mapping_groupedconv2d_tensorcore.py:7-60, mapping_depthwiseconv2d_tensorcore.py:7-48):
    output [N, groups, K/groups, spatial...], the activations' channel index is
    group * (C/groups) + rc (or the group alone when C/groups = 1), the weights are read through a
    reshaping stage.  Lowered to the convolution descriptor with `groups`."""
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    nsp = len(spatial) - 3
    if nsp not in (1, 2, 3) or len(reduce_) not in (nsp, nsp + 1):
        return None
    n_iv, g_iv, k_iv, out_sp = spatial[0], spatial[1], spatial[2], spatial[3:]
    rc = reduce_[0] if len(reduce_) == nsp + 1 else None
    red_sp = reduce_[1:] if rc is not None else reduce_
    variables = [iv.var for iv in spatial + reduce_]
    G, Kg = int(g_iv.dom.extent), int(k_iv.dom.extent)
    Cg = int(rc.dom.extent) if rc is not None else 1

    def try_roles(lx, lw):
        rx, rw = _resolve_dims(lx, variables), _flat_address(lw, variables)
        if rx is None or rw is None or rw[2] != 0:
            return None
        xt, fx = rx
        if len(fx) != nsp + 2 or fx[0] != ({n_iv.var: 1}, 0):
            return None
        want_c = {g_iv.var: Cg}
        if rc is not None:
            want_c[rc.var] = 1
        if fx[1] != (want_c, 0):
            return None
        strides, dils = [], []
        for d in range(nsp):
            coef, const = fx[2 + d]
            if const != 0 or set(coef) - {out_sp[d].var, red_sp[d].var}:
                return None
            strides.append(int(coef.get(out_sp[d].var, 1)))
            dils.append(int(coef.get(red_sp[d].var, 1)))
        # weights: a dense [K][Cg][window...] placeholder, however it is reshaped on the way
        win = [int(r.dom.extent) for r in red_sp]
        trs = 1
        for e in win:
            trs *= e
        want = {g_iv.var: Kg * Cg * trs, k_iv.var: Cg * trs}
        if rc is not None:
            want[rc.var] = trs
        acc = 1
        for r in reversed(red_sp):
            want[r.var] = acc
            acc *= int(r.dom.extent)
        want = {v: c for v, c in want.items() if c != 0 and
                int([iv for iv in spatial + reduce_ if iv.var is v][0].dom.extent) > 1}
        got = {v: c for v, c in rw[1].items()
               if int([iv for iv in spatial + reduce_ if iv.var is v][0].dom.extent) > 1}
        if got != want or _numel(rw[0].shape) != G * Kg * Cg * trs:
            return None
        return xt, rw[0], strides, dils, win

    roles, lx, lw = try_roles(l0, l1), l0, l1
    if roles is None:
        roles, lx, lw = try_roles(l1, l0), l1, l0
    if roles is None:
        return None
    xt, wt, strides, dils, win = roles
    src, pads = _pad_stage(xt)
    xs = [int(s) for s in src.shape]
    if xs[1] != G * Cg:
        raise NoKernelError("activations have %d channels, the compute reads %d groups of %d" % (xs[1], G, Cg))
    for d in range(nsp):
        want = (xs[2 + d] + 2 * pads[d] - ((win[d] - 1) * dils[d] + 1)) // strides[d] + 1
        if int(out_sp[d].dom.extent) != want:
            raise NoKernelError("output extent %d is not what stride / padding / dilation give (%d)"
                                % (int(out_sp[d].dom.extent), want))
    ind, outd = _dtype_pair(lx, lw, main_op.output(0))
    c = _lib.ConvDesc()
    lead = 3 - nsp
    xs5 = xs[:2] + [1] * lead + xs[2:]
    ws5 = [G * Kg, Cg] + [1] * lead + win
    st, pd, dl = [1] * lead + strides, [0] * lead + pads, [1] * lead + dils
    c.N, c.C, c.D, c.H, c.W = xs5
    c.K, _, c.T, c.R, c.S = ws5
    c.stride_d, c.stride_h, c.stride_w = st
    c.pad_d, c.pad_h, c.pad_w = pd
    c.dil_d, c.dil_h, c.dil_w = dl
    c.in_dtype, c.out_dtype = ind, outd
    c.groups = G
    J = xs[0]
    for iv in out_sp:
        J *= int(iv.dom.extent)
    attrs = dict(x_shape=xs, w_shape=[G * Kg, Cg] + win, stride=strides, pad=pads, dil=dils, dtype=lx.dtype,
                 J=J, K_out=G * Kg, K_red=Cg * _numel(win), groups=G)
    kind, code = ("conv2d", _lib.AMOS_OP_CONV2D) if nsp <= 2 else ("conv3d", _lib.AMOS_OP_CONV3D)
    return LoweredOp(kind, code, c, [src, wt], main_op.output(0), attrs)


def _lower_batch_conv(main_op, l0, l1):
    """Convolution with a filter bank per image (benchmark/amos/mapping_batchconv2d_tensorcore.py:7-40:
    Conv[n,k,p,q] = sum Pad[n,rc,...] * B[n,k,rc,rr,rs]): the image index reaches both operands, so it
    is a batch of independent products -- exactly a grouped convolution of ONE image whose
    channels are the N*C channels of all images and whose groups are the images.  The memory of
    A [N][C][...], B [N][K][C][...] and the output [N][K][...] is already that convolution's."""
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    nsp = len(spatial) - 2
    if nsp not in (1, 2, 3) or len(reduce_) != nsp + 1:
        return None
    n_iv, k_iv, out_sp = spatial[0], spatial[1], spatial[2:]
    rc, red_sp = reduce_[0], reduce_[1:]
    variables = [iv.var for iv in spatial + reduce_]

    def try_roles(lx, lw):
        if not isinstance(lw.tensor.op, te.PlaceholderOp) or len(lw.indices) != nsp + 3:
            return None
        if any(i is not v for i, v in zip(lw.indices, [n_iv.var, k_iv.var, rc.var] + [r.var for r in red_sp])):
            return None
        rx = _resolve_dims(lx, variables)
        if rx is None:
            return None
        xt, fx = rx
        if len(fx) != nsp + 2 or fx[0] != ({n_iv.var: 1}, 0) or fx[1] != ({rc.var: 1}, 0):
            return None
        strides, dils = [], []
        for d in range(nsp):
            coef, const = fx[2 + d]
            if const != 0 or set(coef) - {out_sp[d].var, red_sp[d].var}:
                return None
            strides.append(int(coef.get(out_sp[d].var, 1)))
            dils.append(int(coef.get(red_sp[d].var, 1)))
        return xt, strides, dils

    roles, lx, lw = try_roles(l0, l1), l0, l1
    if roles is None:
        roles, lx, lw = try_roles(l1, l0), l1, l0
    if roles is None:
        return None
    xt, strides, dils = roles
    src, pads = _pad_stage(xt)
    xs, ws = [int(e) for e in src.shape], [int(e) for e in lw.tensor.shape]
    N, C, K, win = xs[0], xs[1], ws[1], ws[3:]
    if ws[0] != N or ws[2] != C or int(rc.dom.extent) != C or [int(r.dom.extent) for r in red_sp] != win:
        raise NoKernelError("per-image filters %s do not go with activations %s" % (ws, xs))
    for d in range(nsp):
        want = (xs[2 + d] + 2 * pads[d] - ((win[d] - 1) * dils[d] + 1)) // strides[d] + 1
        if int(out_sp[d].dom.extent) != want:
            raise NoKernelError("output extent %d is not what stride / padding / dilation give (%d)"
                                % (int(out_sp[d].dom.extent), want))
    ind, outd = _dtype_pair(lx, lw, main_op.output(0))
    c = _lib.ConvDesc()
    lead = 3 - nsp
    c.N, c.C, c.D, c.H, c.W = [1, N * C] + [1] * lead + xs[2:]
    c.K, _, c.T, c.R, c.S = [N * K, C] + [1] * lead + win
    c.stride_d, c.stride_h, c.stride_w = [1] * lead + strides
    c.pad_d, c.pad_h, c.pad_w = [0] * lead + pads
    c.dil_d, c.dil_h, c.dil_w = [1] * lead + dils
    c.in_dtype, c.out_dtype = ind, outd
    c.groups = N
    J = _numel([iv.dom.extent for iv in out_sp])
    attrs = dict(x_shape=[1, N * C] + xs[2:], w_shape=[N * K, C] + win, stride=strides, pad=pads, dil=dils,
                 dtype=lx.dtype, J=J, K_out=N * K, K_red=C * _numel(win), groups=N)
    kind, code = ("conv2d", _lib.AMOS_OP_CONV2D) if nsp <= 2 else ("conv3d", _lib.AMOS_OP_CONV3D)
    return LoweredOp(kind, code, c, [src, lw.tensor], main_op.output(0), attrs)


def _lower_capsule_conv(main_op, l0, l1):
    """Convolution whose filters carry a trailing capsule axis
    (benchmark/amos/mapping_capsuleconv2d_tensorcore.py:33-72:
    Out[b,k,h,w,s] = sum padded[b,rc,h*st+rh*dil,w*st+rw*dil] * B[k,rc,rh,rw,s]): (k, s) together are
    the output channels of an ordinary convolution with K * caps filters.  The filters are
    gathered to [K*caps][C][window] in front of the kernel and the result [N][K*caps][spatial] to
    the compute's [N][K][spatial][caps] behind it."""
    spatial, reduce_ = list(main_op.axis), list(main_op.reduce_axis)
    nsp = len(spatial) - 3
    if nsp not in (1, 2, 3) or len(reduce_) != nsp + 1:
        return None
    n_iv, k_iv, out_sp, s_iv = spatial[0], spatial[1], spatial[2:-1], spatial[-1]
    variables = [iv.var for iv in spatial + reduce_]

    def try_roles(lx, lw):
        if not isinstance(lw.tensor.op, te.PlaceholderOp) or len(lw.indices) != nsp + 3:
            return None
        rx = _resolve_dims(lx, variables)
        if rx is None:
            return None
        xt, fx = rx
        if len(fx) != nsp + 2 or fx[0] != ({n_iv.var: 1}, 0):
            return None
        rc = [r for r in reduce_ if fx[1] == ({r.var: 1}, 0)]
        if len(rc) != 1:
            return None
        rc = rc[0]
        strides, dils, red_sp = [], [], []
        for d in range(nsp):
            coef, const = fx[2 + d]
            rv = [r for r in reduce_ if r.var in coef and r is not rc]
            if const != 0 or len(rv) != 1 or set(coef) - {out_sp[d].var, rv[0].var}:
                return None
            red_sp.append(rv[0])
            strides.append(int(coef.get(out_sp[d].var, 1)))
            dils.append(int(coef[rv[0].var]))
        want = [k_iv.var, rc.var] + [r.var for r in red_sp] + [s_iv.var]
        if any(i is not v for i, v in zip(lw.indices, want)):
            return None
        return xt, rc, red_sp, strides, dils

    roles, lx, lw = try_roles(l0, l1), l0, l1
    if roles is None:
        roles, lx, lw = try_roles(l1, l0), l1, l0
    if roles is None:
        return None
    xt, rc, red_sp, strides, dils = roles
    src, pads = _pad_stage(xt)
    xs, ws = [int(e) for e in src.shape], [int(e) for e in lw.tensor.shape]
    N, C = xs[0], xs[1]
    K, win, caps = ws[0], ws[2:-1], ws[-1]
    if ws[1] != C or int(rc.dom.extent) != C or [int(r.dom.extent) for r in red_sp] != win or \
            int(s_iv.dom.extent) != caps or int(k_iv.dom.extent) != K:
        raise NoKernelError("capsule filters %s do not go with activations %s" % (ws, xs))
    osp = [int(iv.dom.extent) for iv in out_sp]
    for d in range(nsp):
        want = (xs[2 + d] + 2 * pads[d] - ((win[d] - 1) * dils[d] + 1)) // strides[d] + 1
        if osp[d] != want:
            raise NoKernelError("output extent %d is not what stride / padding / dilation give (%d)" % (osp[d], want))
    ind, outd = _dtype_pair(lx, lw, main_op.output(0))
    Kc, trs, pq = K * caps, _numel(win), _numel(osp)
    c = _lib.ConvDesc()
    lead = 3 - nsp
    c.N, c.C, c.D, c.H, c.W = [N, C] + [1] * lead + xs[2:]
    c.K, _, c.T, c.R, c.S = [Kc, C] + [1] * lead + win
    c.stride_d, c.stride_h, c.stride_w = [1] * lead + strides
    c.pad_d, c.pad_h, c.pad_w = [0] * lead + pads
    c.dil_d, c.dil_h, c.dil_w = [1] * lead + dils
    c.in_dtype, c.out_dtype = ind, outd
    attrs = dict(x_shape=xs, w_shape=[Kc, C] + win, stride=strides, pad=pads, dil=dils, dtype=lx.dtype,
                 J=N * pq, K_out=Kc, K_red=C * trs)
    kind, code = ("conv2d", _lib.AMOS_OP_CONV2D) if nsp <= 2 else ("conv3d", _lib.AMOS_OP_CONV3D)
    low = LoweredOp(kind, code, c, [src, lw.tensor], main_op.output(0), attrs)
    # filters: element (k*caps + s, c, window...) of the kernel's operand is B[k][c][window...][s]
    w_tabs = [[(i // caps) * (C * trs * caps) + i % caps for i in range(Kc)], [cc * trs * caps for cc in range(C)]]
    stride = trs
    for e in win:
        stride //= e
        w_tabs.append([i * stride * caps for i in range(e)])
    low.gathers[1] = OperandView(lw.tensor, [Kc, C] + win, w_tabs, lw.tensor.dtype)
    # result: Out[n][k][spatial...][s] is element (n, k*caps + s, spatial...) of what the kernel writes
    o_tabs = [[n * Kc * pq for n in range(N)], [k * caps * pq for k in range(K)]]
    stride = pq
    for e in osp:
        stride //= e
        o_tabs.append([i * stride for i in range(e)])
    o_tabs.append([sx * pq for sx in range(caps)])
    low.out_view = OperandView(None, [N, K] + osp + [caps], o_tabs, main_op.output(0).dtype)
    return low


def lower_main_op(main_op, target_dag=None):
    """ComputeOp that matched a GEMM-like intrinsic -> LoweredOp; with the compute DAG it
    belongs to, an element-wise addition behind it is fused into the kernel"""
    low = _lower_main_op(main_op)
    return _fuse_tail(low, main_op, target_dag) if target_dag is not None else low


def _lower_main_op(main_op):
    l0, l1 = _product_loads(main_op)
    iters = list(main_op.axis) + list(main_op.reduce_axis)
    variables = [iv.var for iv in iters]
    forms0 = [te.affine_form(i, variables) for i in l0.indices]
    forms1 = [te.affine_form(i, variables) for i in l1.indices]
    for fn in (_lower_strided_gemm, _lower_grouped_conv, _lower_batch_conv, _lower_capsule_conv):
        low = fn(main_op, l0, l1)
        if low is not None:
            return low
    for fn in (_lower_gemm, _lower_conv):
        low = fn(main_op, l0, l1, iters, forms0, forms1)
        if low is not None:
            return low
    raise NoKernelError("access pattern of %s is neither GEMM, batched GEMM, NCHW conv2d nor NCDHW conv3d"
                        % main_op.name)
