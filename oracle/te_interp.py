"""TEST INFRASTRUCTURE: brute-force evaluator of mini-TE computes (tiny shapes only).

Evaluates a compute exactly as written -- loops over the output axes, then over the reduce
axes in their declared order, exact integer / float64 arithmetic -- so that tests can check
that lowering a compute to an operator descriptor kept its meaning."""
import itertools

import numpy as np

from amos_amd import te


def evaluate(tensor, feeds, cache=None):
    """tensor -> numpy array (float64 / int64); feeds maps placeholder name -> numpy array"""
    cache = {} if cache is None else cache
    if id(tensor) in cache:
        return cache[id(tensor)]
    op = tensor.op
    if isinstance(op, te.PlaceholderOp):
        arr = np.asarray(feeds[tensor.name])
        out = arr.astype(np.int64 if arr.dtype.kind in "iu" else np.float64)
        cache[id(tensor)] = out
        return out
    inputs = {id(t): evaluate(t, feeds, cache) for t in op.input_tensors}
    shape = [int(s) for s in tensor.shape]
    out = np.zeros(shape, dtype=np.int64 if tensor.dtype.startswith("int") else np.float64)
    env = {}

    def ev(e):
        if isinstance(e, te.IntImm) or isinstance(e, te.FloatImm):
            return e.value
        if isinstance(e, te.Var):
            return env[id(e)]
        if isinstance(e, te.Add): return ev(e.a) + ev(e.b)
        if isinstance(e, te.Sub): return ev(e.a) - ev(e.b)
        if isinstance(e, te.Mul): return ev(e.a) * ev(e.b)
        if isinstance(e, te.FloorDiv): return ev(e.a) // ev(e.b)
        if isinstance(e, te.FloorMod): return ev(e.a) % ev(e.b)
        if isinstance(e, te.Cmp):
            a, b = ev(e.a), ev(e.b)
            return {">=": a >= b, ">": a > b, "<=": a <= b, "<": a < b, "==": a == b}[e.op]
        if isinstance(e, te.And): return all(ev(t) for t in e.terms)
        if isinstance(e, te.Cast): return ev(e.value)
        if isinstance(e, te.Select): return ev(e.then_value) if ev(e.cond) else ev(e.else_value)
        if isinstance(e, te.ProducerLoad):
            return inputs[id(e.tensor)][tuple(int(ev(i)) for i in e.indices)]
        if isinstance(e, te.Reduce):
            acc = 0
            for vals in itertools.product(*[range(int(a.dom.extent)) for a in e.axis]):
                for a, v in zip(e.axis, vals):
                    env[id(a.var)] = v
                acc = acc + ev(e.source)
            return acc
        raise TypeError("cannot evaluate %r" % (e,))

    for idx in itertools.product(*[range(s) for s in shape]):
        for a, v in zip(op.axis, idx):
            env[id(a.var)] = v
        out[idx] = ev(op.body[0])
    cache[id(tensor)] = out
    return out
