"""Matching a compute against the registered intrinsics.

Mirrors python/tvm/auto_tensorize/tensorization_phases/intrin_match.py: IntrinMatchResult
(:11-68), intrinsic_match with its sort of the match points (:83-97), get_match_results
(:168-181).  The match itself runs in C++ (amos_match in libamos_mi355x.so), fed with the
body structure and the affine index rows of both computes.
"""
import ctypes

from .. import _lib, te
from .hw_abs_dag import query_hw_abs_dag
from .hw_abstraction import ComputeDAG

_DTYPE_CODE = {"float16": 1, "bfloat16": 2, "int8": 3, "float32": 4, "int32": 5, "float64": 6,
               "int64": 7, "uint8": 8, "bool": 9}
_KIND = {"reduce": 1, "cast": 2, "mul": 3, "add": 4, "sub": 5, "load": 6, "select": 7, "const": 8,
         "other": 9}


class IntrinMatchResult(object):
    """
    hw_abs_dag: HardwareAbstractionDAG   the matched intrinsic DAG
    compute_key, shape_key: str
    main_op_map: {intrinsic main op: target op}
    axis_map: {intrinsic IterVar: [target IterVar per match point]}
    target_dag, intrin_dag: ComputeDAG
    """

    def __init__(self, hw_abs_dag, compute_key, shape_key, main_op_map, elem_op_map, axis_map,
                 target_dag, intrin_dag):
        self.hw_abs_dag = hw_abs_dag
        self.compute_key = compute_key
        self.shape_key = shape_key
        self.main_op_map = main_op_map
        self.elem_op_map = elem_op_map
        self.axis_map = axis_map
        self.target_dag = target_dag
        self.intrin_dag = intrin_dag

    def get_hw_abs_dag(self): return self.hw_abs_dag
    def get_compute_key(self): return self.compute_key
    def get_shape_key(self): return self.shape_key
    def get_main_op_map(self): return self.main_op_map
    def get_elem_op_map(self): return self.elem_op_map
    def get_target_dag(self): return self.target_dag
    def get_intrin_dag(self): return self.intrin_dag

    def __str__(self):
        return "MatchResult(hw_abs_dag:%s, compute:%s, shape:%s)" % (
            self.hw_abs_dag.get_name(), self.compute_key, self.shape_key)


class _ComputeC(object):
    """keeps the ctypes arrays of an amos_compute_t alive"""

    def __init__(self, op):
        iters = list(op.axis) + list(op.reduce_axis)
        variables = [iv.var for iv in iters]
        tokens, loads = [], []

        def tok(kind, dtype):
            tokens.append((_KIND[kind] << 8) | _DTYPE_CODE.get(dtype, 15))

        def walk(e):
            if isinstance(e, te.Reduce):
                tok("reduce", e.dtype); walk(e.source)
            elif isinstance(e, te.Cast):
                tok("cast", e.dtype); walk(e.value)
            elif isinstance(e, te.Mul):
                tok("mul", e.dtype); walk(e.a); walk(e.b)
            elif isinstance(e, te.Add):
                tok("add", e.dtype); walk(e.a); walk(e.b)
            elif isinstance(e, te.Sub):
                tok("sub", e.dtype); walk(e.a); walk(e.b)
            elif isinstance(e, te.ProducerLoad):
                tok("load", e.dtype); loads.append(e)
            elif isinstance(e, te.Select):
                tok("select", e.dtype); walk(e.then_value); walk(e.else_value)
            elif isinstance(e, (te.IntImm, te.FloatImm)):
                tok("const", e.dtype)
            else:
                tok("other", getattr(e, "dtype", ""))

        walk(op.body[0])
        n = len(iters)
        rows = []
        for ld in loads:
            for idx in ld.indices:
                form = te.affine_form(idx, variables)
                if form is None:
                    # opaque index: mark every variable that occurs in it
                    occurs = set()
                    _collect_vars(idx, occurs)
                    rows.extend([1 if id(v) in occurs else 0 for v in variables] + [0, 0])
                else:
                    coef, const = form
                    rows.extend([coef.get(v, 0) for v in variables] + [const, 1])
        self.iters = iters
        self.loads = loads
        self._tokens = (ctypes.c_int32 * max(1, len(tokens)))(*tokens)
        self._kinds = (ctypes.c_int32 * n)(*[iv.iter_type for iv in iters])
        self._extents = (ctypes.c_int64 * n)(*[int(iv.dom.extent) for iv in iters])
        self._ndim = (ctypes.c_int32 * max(1, len(loads)))(*[len(ld.indices) for ld in loads])
        self._coeffs = (ctypes.c_int64 * max(1, len(rows)))(*rows)
        self.c = _lib.ComputeC(len(tokens), self._tokens, n, self._kinds, self._extents, len(loads),
                               self._ndim, self._coeffs)


def _collect_vars(e, out):
    if isinstance(e, te.Var):
        out.add(id(e))
    for attr in ("a", "b", "value", "cond", "then_value", "else_value", "source"):
        child = getattr(e, attr, None)
        if isinstance(child, te.Expr):
            _collect_vars(child, out)
    for child in getattr(e, "terms", []) or []:
        _collect_vars(child, out)
    for child in getattr(e, "indices", []) or []:
        _collect_vars(child, out)


def intrinsic_match(target_op, intrin_op):
    """match points of one target ComputeOp: list of {target IterVar: intrinsic IterVar},
    sorted by the sorted set of target axis names (reference: intrin_match.py:88-97)"""
    if not isinstance(target_op, te.ComputeOp):
        return []
    tgt, itr = _ComputeC(target_op), _ComputeC(intrin_op)
    ni = len(itr.iters)
    cap = 4096
    buf = (ctypes.c_int32 * (cap * ni))()
    n = _lib.check(_lib.load().amos_match(ctypes.byref(tgt.c), ctypes.byref(itr.c), buf, cap))
    if n > cap:
        raise RuntimeError("more than %d match points" % cap)
    points = []
    for p in range(n):
        points.append({tgt.iters[buf[p * ni + a]]: itr.iters[a] for a in range(ni)})

    def key(point):
        return str(list(sorted(tuple(set(iv.var.name for iv in point)))))

    return sorted(points, key=key)


def intrinsic_multi_match(target_dag, intrin_dag, main_op):
    """every ComputeOp of the target DAG is tried as the main op (intrin_match.py:105-114)"""
    results = {}
    for op in target_dag.op_lst:
        points = intrinsic_match(op, main_op)
        if points:
            results[op] = points
    return results


def get_match_result_with_hw_abs_dag(target_dag, hw_abs_dag, compute_key, shape_key):
    intrin_dag, main_tensors = hw_abs_dag.get_effective_compute_dag(compute_key, shape_key)
    assert len(main_tensors) == 1
    main_op = main_tensors[0].op
    raw_match = intrinsic_multi_match(target_dag, intrin_dag, main_op)
    match_results = []
    for top, match_points in raw_match.items():
        axis_map = {iiv: [] for iiv in list(main_op.axis) + list(main_op.reduce_axis)}
        for point in match_points:
            for tiv, iiv in point.items():
                axis_map[iiv].append(tiv)
        match_results.append(IntrinMatchResult(hw_abs_dag, compute_key, shape_key, {main_op: top}, {},
                                               axis_map, target_dag, intrin_dag))
    return match_results


def get_match_results(target_dag, target):
    """all (DAG class x compute key x shape key) matches of a compute for a target"""
    assert isinstance(target_dag, ComputeDAG)
    ret = []
    for hw_abs_dag_cls in query_hw_abs_dag(target):
        hw_abs_dag = hw_abs_dag_cls()
        for compute_key in hw_abs_dag.get_all_compute_keys():
            for shape_key in hw_abs_dag.get_all_shape_keys():
                ret.extend(get_match_result_with_hw_abs_dag(target_dag, hw_abs_dag, compute_key, shape_key))
    return ret
