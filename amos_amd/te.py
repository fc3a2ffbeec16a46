"""A small tensor-expression front end: just enough of TVM's `te` / `tir` surface to
*describe* the computes the auto-tensorize path handles (GEMM, batched GEMM, conv2d,
conv3d and their padding stages) so that they can be matched against an intrinsic.

Nothing here executes a compute; expressions are inert trees.  The spelling follows the
reference's scripts (reference: benchmark/amos/mapping_gemm_tensorcore.py:7-15,
benchmark/amos/mapping_conv2d_tensorcore.py:7-42):

    A = te.placeholder([M, K], dtype="float16", name="A")
    rk = te.reduce_axis([0, K], name="k")
    C = te.compute([M, N], lambda i, j: te.sum((A[i, rk] * B[rk, j]).astype("float32"), axis=rk))
"""
import inspect
from numbers import Integral, Real

# iteration kinds, numbered as in TVM's IterVarType
DATA_PAR = 0
COMM_REDUCE = 2


class Range(object):
    def __init__(self, min_value, extent):
        self.min = IntImm(int(min_value))
        self.extent = IntImm(int(extent))


class Expr(object):
    dtype = "int32"

    # arithmetic -------------------------------------------------------------------
    def __add__(self, o): return Add(self, const_like(o, self))
    def __radd__(self, o): return Add(const_like(o, self), self)
    def __sub__(self, o): return Sub(self, const_like(o, self))
    def __rsub__(self, o): return Sub(const_like(o, self), self)
    def __mul__(self, o): return Mul(self, const_like(o, self))
    def __rmul__(self, o): return Mul(const_like(o, self), self)
    def __floordiv__(self, o): return FloorDiv(self, const_like(o, self))
    def __mod__(self, o): return FloorMod(self, const_like(o, self))
    def __neg__(self): return Sub(const_like(0, self), self)
    # comparisons ------------------------------------------------------------------
    def __ge__(self, o): return Cmp(">=", self, const_like(o, self))
    def __gt__(self, o): return Cmp(">", self, const_like(o, self))
    def __le__(self, o): return Cmp("<=", self, const_like(o, self))
    def __lt__(self, o): return Cmp("<", self, const_like(o, self))
    def equal(self, o): return Cmp("==", self, const_like(o, self))
    # `a == b` builds the comparison, as in TVM; asked for its truth value (tuple, set and dict
    # comparisons do) it answers whether both sides are the same object
    def __eq__(self, o): return _EqCmp(self, const_like(o, self))

    def astype(self, dtype):
        return self if dtype == self.dtype else Cast(dtype, self)

    def __bool__(self):
        raise TypeError("a tensor expression has no truth value; use tir.all / tir.if_then_else")

    __hash__ = object.__hash__


def const_like(v, like):
    if isinstance(v, Expr):
        return v
    if isinstance(v, IterVar):
        return v.var
    if isinstance(v, bool):
        return IntImm(int(v), "bool")
    if isinstance(v, Integral):
        return IntImm(int(v), like.dtype if like.dtype.startswith("int") else "int32")
    if isinstance(v, Real):
        return FloatImm(float(v), like.dtype if like.dtype.startswith("float") else "float32")
    raise TypeError("cannot use %r in a tensor expression" % (v,))


class IntImm(Expr):
    def __init__(self, value, dtype="int32"):
        self.value = int(value)
        self.dtype = dtype

    def __int__(self): return self.value
    def __index__(self): return self.value
    def __repr__(self): return str(self.value)


class FloatImm(Expr):
    def __init__(self, value, dtype="float32"):
        self.value = float(value)
        self.dtype = dtype

    def __repr__(self): return "%sf" % self.value


class Var(Expr):
    def __init__(self, name, dtype="int32"):
        self.name = name
        self.dtype = dtype

    def __repr__(self): return self.name


class IterVar(object):
    """An iteration variable with its range; arithmetic goes through `.var`."""

    def __init__(self, dom, name, iter_type=DATA_PAR):
        if isinstance(dom, Range):
            self.dom = dom
        else:
            lo, hi = dom
            self.dom = Range(int(lo), int(hi) - int(lo))
        self.var = Var(name) if isinstance(name, str) else name
        self.iter_type = iter_type

    def __repr__(self): return "iter_var(%s, range(min=%d, ext=%d))" % (self.var.name, int(self.dom.min), int(self.dom.extent))

    # let an IterVar stand in an index expression, as TVM does
    def __add__(self, o): return self.var + o
    def __radd__(self, o): return o + self.var
    def __sub__(self, o): return self.var - o
    def __rsub__(self, o): return o - self.var
    def __mul__(self, o): return self.var * o
    def __rmul__(self, o): return o * self.var
    def __floordiv__(self, o): return self.var // o
    def __mod__(self, o): return self.var % o
    def __ge__(self, o): return self.var >= o
    def __gt__(self, o): return self.var > o
    def __le__(self, o): return self.var <= o
    def __lt__(self, o): return self.var < o
    __hash__ = object.__hash__


class _Binary(Expr):
    op = "?"

    def __init__(self, a, b):
        self.a, self.b = a, b
        self.dtype = a.dtype

    def __repr__(self): return "(%r %s %r)" % (self.a, self.op, self.b)


class Add(_Binary): op = "+"
class Sub(_Binary): op = "-"
class Mul(_Binary): op = "*"
class FloorDiv(_Binary): op = "//"
class FloorMod(_Binary): op = "%"


class Cmp(Expr):
    def __init__(self, op, a, b):
        self.op, self.a, self.b = op, a, b
        self.dtype = "bool"

    def __repr__(self): return "(%r %s %r)" % (self.a, self.op, self.b)


class _EqCmp(Cmp):
    def __init__(self, a, b):
        Cmp.__init__(self, "==", a, b)

    def __bool__(self):
        return self.a is self.b


class And(Expr):
    def __init__(self, terms):
        self.terms = list(terms)
        self.dtype = "bool"

    def __repr__(self): return "(" + " && ".join(repr(t) for t in self.terms) + ")"


class Cast(Expr):
    def __init__(self, dtype, value):
        self.dtype = dtype
        self.value = value

    def __repr__(self): return "%s(%r)" % (self.dtype, self.value)


class Select(Expr):
    """tir.if_then_else(cond, then, else)"""

    def __init__(self, cond, then_value, else_value):
        self.cond, self.then_value, self.else_value = cond, then_value, else_value
        self.dtype = then_value.dtype

    def __repr__(self): return "if_then_else(%r, %r, %r)" % (self.cond, self.then_value, self.else_value)


class ProducerLoad(Expr):
    def __init__(self, tensor, indices):
        self.tensor = tensor
        self.indices = list(indices)
        self.dtype = tensor.dtype

    def __repr__(self): return "%s[%s]" % (self.tensor.name, ", ".join(repr(i) for i in self.indices))


class Reduce(Expr):
    """te.sum(source, axis): init 0, then += in the declared axis order."""

    def __init__(self, source, axis):
        self.source = source
        self.axis = list(axis)
        self.dtype = source.dtype

    def __repr__(self): return "reduce(sum, %r, axis=[%s])" % (self.source, ", ".join(a.var.name for a in self.axis))


# ---- operations and tensors -------------------------------------------------------------
class Operation(object):
    def output(self, index):
        assert index == 0
        return self._output

    __hash__ = object.__hash__


class PlaceholderOp(Operation):
    def __init__(self, name, shape, dtype):
        self.name = name
        self.input_tensors = []
        self._output = Tensor(shape, dtype, name, self)

    def __repr__(self): return "placeholder(%s)" % self.name


class ComputeOp(Operation):
    def __init__(self, name, axis, reduce_axis, body, shape, dtype):
        self.name = name
        self.axis = list(axis)
        self.reduce_axis = list(reduce_axis)
        self.body = [body]
        seen, inputs = set(), []
        for ld in collect_loads(body):
            if id(ld.tensor) not in seen:
                seen.add(id(ld.tensor))
                inputs.append(ld.tensor)
        self.input_tensors = inputs
        self._output = Tensor(shape, dtype, name, self)

    def __repr__(self): return "compute(%s)" % self.name


class Tensor(object):
    def __init__(self, shape, dtype, name, op):
        self.shape = [s if isinstance(s, IntImm) else IntImm(int(s)) for s in shape]
        self.dtype = dtype
        self.name = name
        self.op = op

    def __getitem__(self, indices):
        if not isinstance(indices, tuple):
            indices = (indices,)
        if len(indices) != len(self.shape):
            raise ValueError("%s has %d dimensions, indexed with %d" % (self.name, len(self.shape), len(indices)))
        return ProducerLoad(self, [const_like(i, IntImm(0)) for i in indices])

    def __call__(self, *indices):
        return self[tuple(indices)]

    @property
    def ndim(self): return len(self.shape)

    def __repr__(self):
        return "Tensor(shape=[%s], op.name=%s)" % (", ".join(str(int(s)) for s in self.shape), self.name)

    __hash__ = object.__hash__


def collect_loads(expr):
    """ProducerLoads of an expression in evaluation (left to right) order"""
    out = []

    def walk(e):
        if isinstance(e, ProducerLoad):
            out.append(e)
            for i in e.indices:
                walk(i)
        elif isinstance(e, _Binary) or isinstance(e, Cmp):
            walk(e.a)
            walk(e.b)
        elif isinstance(e, And):
            for t in e.terms:
                walk(t)
        elif isinstance(e, Cast):
            walk(e.value)
        elif isinstance(e, Select):
            walk(e.cond)
            walk(e.then_value)
            walk(e.else_value)
        elif isinstance(e, Reduce):
            walk(e.source)

    walk(expr)
    return out


# ---- the te.* functions -----------------------------------------------------------------
def placeholder(shape, dtype="float32", name="placeholder"):
    return PlaceholderOp(name, list(shape), dtype).output(0)


def reduce_axis(dom, name="rv"):
    return IterVar(dom, name, COMM_REDUCE)


def thread_axis(*args, **kwargs):
    raise NotImplementedError("schedules are not expressed in this front end")


def sum(expr, axis):  # noqa: A001 - mirrors te.sum
    axes = list(axis) if isinstance(axis, (list, tuple)) else [axis]
    for a in axes:
        if not isinstance(a, IterVar) or a.iter_type != COMM_REDUCE:
            raise TypeError("te.sum needs reduce axes made by te.reduce_axis")
    return Reduce(expr, axes)


_AXIS_NAMES = "ijklmnopqrstuvwxyz"


def compute(shape, fcompute, name="compute", tag="", attrs=None):
    shape = [int(s) for s in shape]
    sig = inspect.signature(fcompute).parameters
    params = list(sig)
    if len(params) == 1 and sig[params[0]].kind == inspect.Parameter.VAR_POSITIONAL:
        params = ["i%d" % d for d in range(len(shape))]     # lambda *indices, as TVM names them
    if len(params) != len(shape):
        raise ValueError("fcompute takes %d indices for a %d-d output" % (len(params), len(shape)))
    axis = [IterVar((0, ext), pname) for pname, ext in zip(params, shape)]
    body = fcompute(*[iv.var for iv in axis])
    if not isinstance(body, Expr):
        body = const_like(body, FloatImm(0.0))
    red = body.axis if isinstance(body, Reduce) else []
    return ComputeOp(name, axis, red, body, shape, body.dtype).output(0)


class Schedule(object):
    """Placeholder for te.create_schedule: the kernel schedule is a KernelConfig, not a TE schedule."""

    def __init__(self, ops):
        self.outputs = list(ops)
        self.kernel_config = None


def create_schedule(ops):
    return Schedule(ops if isinstance(ops, (list, tuple)) else [ops])


# ---- the tir.* helpers the computes use ----------------------------------------------------
class _Tir(object):
    IterVar = IterVar
    Var = Var

    @staticmethod
    def if_then_else(cond, then_value, else_value):
        then_value = const_like(then_value, FloatImm(0.0))
        else_value = const_like(else_value, then_value)
        return Select(cond, then_value, else_value)

    @staticmethod
    def all(*conds):
        return And(conds)

    @staticmethod
    def const(value, dtype="float32"):
        if dtype.startswith("int") or dtype.startswith("uint") or dtype == "bool":
            return IntImm(int(value), dtype)
        return FloatImm(float(value), dtype)


tir = _Tir()
if_then_else = tir.if_then_else
globals()["all"] = tir.all      # te.all(...), as tvm.te.all


# ---- affine views of index expressions -------------------------------------------------------
def affine_form(expr, variables):
    """index expression -> ({variable: integer coefficient}, constant), or None if not affine in
    `variables` (a list of Var)."""
    ids = {id(v): v for v in variables}

    def walk(e):
        if isinstance(e, IntImm):
            return {}, e.value
        if isinstance(e, Var):
            if id(e) in ids:
                return {id(e): 1}, 0
            return None
        if isinstance(e, (Add, Sub)):
            a, b = walk(e.a), walk(e.b)
            if a is None or b is None:
                return None
            sign = 1 if isinstance(e, Add) else -1
            coef = dict(a[0])
            for k, v in b[0].items():
                coef[k] = coef.get(k, 0) + sign * v
            return coef, a[1] + sign * b[1]
        if isinstance(e, Mul):
            a, b = walk(e.a), walk(e.b)
            if a is None or b is None:
                return None
            if not a[0]:
                return {k: v * a[1] for k, v in b[0].items()}, a[1] * b[1]
            if not b[0]:
                return {k: v * b[1] for k, v in a[0].items()}, a[1] * b[1]
            return None
        if isinstance(e, Cast):
            return walk(e.value)
        return None

    res = walk(expr)
    if res is None:
        return None
    return {ids[k]: v for k, v in res[0].items() if v != 0}, res[1]
