"""`tvm`-shaped facade so that a script written against the reference keeps its shape:

    import amos_amd.tvm as tvm
    from amos_amd.tvm import auto_tensorize as at

    A = tvm.te.placeholder(...); C = tvm.te.compute(...)
    result = at.auto_tensorize(at.compute_dag_from_tensors([C]), "hip", "gemm.log", measure_opt)
    sch, args = at.get_schedule(result.sch_app, result.params)
    func = tvm.build(sch, args, "hip"); func(a, b, c)

Only the names the auto-tensorize scripts use exist (te, tir, auto_tensorize, build, lower, nd,
context, testing); this is not TVM.
"""
import numpy as _np

from .. import auto_tensorize, te  # noqa: F401
from ..auto_tensorize.runtime import array as _array, build, context  # noqa: F401
from ..te import tir  # noqa: F401


class _ND(object):
    array = staticmethod(_array)


nd = _ND()


def gpu(dev_id=0):
    return context("hip", dev_id)


def lower(sch, args, simple_mode=True):
    """one-line description of what will run (there is no TIR to print)"""
    low = getattr(sch, "lowered", None)
    return "kernel: %s\nconfig: %s" % (low, getattr(sch, "kernel_config", None))


class _Testing(object):
    @staticmethod
    def assert_allclose(actual, desired, rtol=1e-7, atol=1e-7):
        _np.testing.assert_allclose(actual, desired, rtol=rtol, atol=atol)


testing = _Testing()
