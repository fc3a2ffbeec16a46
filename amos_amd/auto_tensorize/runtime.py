"""The runnable module: what `build(sch, args, target)` returns.

Stands where tvm.build + tvm.runtime.Module stand in the reference
(python/tvm/auto_tensorize/auto_tensorize.py:294-301, src/runtime/cuda/cuda_module.cc:105-172):
`func(*arrays)` takes the arrays in `inputs + outputs` order, launches on the current
stream and returns without synchronising; `time_evaluator` follows
src/runtime/rpc/rpc_module.cc:341-399.  Arrays are device tensors; there is no host path.
"""
import numpy as np
import torch

from .. import ops
from .measure import _TORCH_DTYPE


class NDArray(object):
    """device array with the asnumpy() / shape / dtype face of tvm.nd.NDArray"""

    def __init__(self, tensor, dtype_name):
        self.tensor = tensor
        self.dtype = dtype_name

    @property
    def shape(self): return tuple(self.tensor.shape)

    def asnumpy(self):
        t = self.tensor
        if t.dtype == torch.bfloat16:
            return t.float().cpu().numpy()
        return t.cpu().numpy()

    numpy = asnumpy


class Context(object):
    def __init__(self, target, dev_id=0):
        self.target, self.dev_id = target, dev_id
        self.device = torch.device("cuda", dev_id)

    def sync(self):
        torch.cuda.synchronize(self.device)


def context(target="hip", dev_id=0):
    return Context(target, dev_id)


def array(np_array, ctx=None, dtype=None):
    """host numpy array -> device array; dtype names 'float16', 'bfloat16', 'int8', 'float32', 'int32'"""
    if not torch.cuda.is_available():
        raise RuntimeError("device arrays need a GPU: no HIP device is visible")
    dev = ctx.device if ctx is not None else torch.device("cuda", 0)
    name = dtype or str(np_array.dtype)
    if name == "bfloat16":
        t = torch.from_numpy(np.ascontiguousarray(np_array, dtype=np.float32)).to(dev).to(torch.bfloat16)
    else:
        t = torch.from_numpy(np.ascontiguousarray(np_array)).to(dev)
        if name in _TORCH_DTYPE and t.dtype != _TORCH_DTYPE[name]:
            t = t.to(_TORCH_DTYPE[name])
    return NDArray(t, name)


class _Source(object):
    def __init__(self, mod): self.mod = mod

    def get_source(self):
        return self.mod.get_source()


class TimeResult(object):
    def __init__(self, results):
        self.results = list(results)
        self.mean = sum(results) / len(results)


class Module(object):
    entry_name = "default_function"

    def __init__(self, lowered, params, arg_tensors):
        self.lowered = lowered
        self.params = params
        # positions of (in0, in1, out[, added tensor of a fused tail]) among the caller's arguments
        ids = [id(t) for t in arg_tensors]
        consts = getattr(lowered, "constants", {})
        computed = getattr(lowered, "computed", {})
        try:
            # (an operand computed from its indices alone is held by the module, not passed; one
            # computed element-wise from placeholders is made per call from those)
            self.arg_index = [None if (k in consts or k in computed) else ids.index(id(lowered.inputs[k]))
                              for k in (0, 1)]
            self._computed_args = {k: [ids.index(id(t)) for t in st.inputs] for k, st in computed.items()}
            self.arg_index.append(ids.index(id(lowered.output)))
            if getattr(lowered, "add_input", None) is not None:
                self.arg_index.append(ids.index(id(lowered.add_input)))
        except ValueError:
            raise ValueError("build() args must hold the compute's inputs and its output tensor")
        self.imported_modules = [_Source(self)]
        self._gathers = {}     # operand position -> (ops.Gather, materialised operand), made on first use
        self._constants = {}   # operand position -> device tensor of a constant operand
        self._out_gather = None   # (ops.Gather, the kernel's own output buffer) where the result is reordered
        self._eltwise = {}        # operand position -> (ops.Eltwise, its result buffer)

    def _kernel_inputs(self, in0, in1):
        """the operands the kernel reads: the caller's arrays, or what the stages in front of an
        operand make of them (materialised into a buffer the module keeps)"""
        ins = [in0, in1]
        for pos, view in getattr(self.lowered, "gathers", {}).items():
            if pos not in self._gathers:
                g = ops.Gather(view.shape, view.tables, _TORCH_DTYPE[view.dtype], ins[pos].numel(), ins[pos].device)
                self._gathers[pos] = (g, torch.empty(g.out_shape, dtype=g.dtype, device=ins[pos].device))
            g, buf = self._gathers[pos]
            ins[pos] = g(ins[pos].contiguous(), buf)
        return ins

    def _computed_operand(self, k, arrays):
        """(stage, its input tensors, its result buffer) of an operand that is an element-wise
        function of the caller's arrays"""
        stage = self.lowered.computed[k]
        ins = []
        for i in self._computed_args[k]:
            a = arrays[i]
            ins.append((a.tensor if isinstance(a, NDArray) else a).contiguous())
        if k not in self._eltwise:
            e = ops.Eltwise(stage.program, len(ins), ins[0].dtype, ins[0].numel())
            self._eltwise[k] = (e, torch.empty_like(ins[0]))
        e, buf = self._eltwise[k]
        return e, ins, buf

    def _pick(self, arrays):
        need = max([i for i in self.arg_index if i is not None] + [i for v in self._computed_args.values() for i in v])
        if len(arrays) <= need:
            raise ValueError("expected %d arrays (inputs + outputs)" % (need + 1))
        out = []
        for k, i in enumerate(self.arg_index):
            if i is None and k in self._computed_args:
                e, ins, buf = self._computed_operand(k, arrays)
                out.append(e(ins, buf))
                continue
            if i is None:
                if k not in self._constants:
                    dev = [a for a in arrays if isinstance(a, (NDArray, torch.Tensor))][0]
                    dev = (dev.tensor if isinstance(dev, NDArray) else dev).device
                    self._constants[k] = torch.from_numpy(self.lowered.constants[k]).to(dev)
                out.append(self._constants[k])
                continue
            a = arrays[i]
            out.append(a.tensor if isinstance(a, NDArray) else a)
        passed = [(k, t) for k, (t, i) in enumerate(zip(out, self.arg_index)) if i is not None]
        for k, t in passed:     # extents and element types of every array first, then where they live
            self._check_array(k, t, placement=False)
        for k, t in passed:
            self._check_array(k, t, placement=True)
        return out

    def _check_array(self, k, t, placement):
        """The kernels take raw pointers: an array that is not the tensor the compute declares
        (its extents, its element type, on a device, dense) is refused before any launch, as the
        reference's argument binder does at call time."""
        lw = self.lowered
        decl = lw.inputs[k] if k < 2 else lw.output if k == 2 else lw.add_input
        what = ("first operand", "second operand", "output", "added operand")[k]
        if not isinstance(t, torch.Tensor):
            raise ValueError("%s %s must be a device array, got %s" % (what, decl.name, type(t).__name__))
        shape = tuple(int(e) for e in decl.shape)
        if tuple(t.shape) != shape or t.dtype != _TORCH_DTYPE[decl.dtype]:
            raise ValueError("%s %s is declared %s %s, the array passed is %s %s"
                             % (what, decl.name, decl.dtype, shape, str(t.dtype).replace("torch.", ""), tuple(t.shape)))
        if not placement:
            return
        if not t.is_cuda:
            raise ValueError("%s %s must be a device array, got one on %s" % (what, decl.name, t.device))
        if not t.is_contiguous():
            raise ValueError("%s %s must be a dense (contiguous) array" % (what, decl.name))

    def _kernel_output(self, out):
        """where the kernel writes: the caller's array, or a buffer of the module's from which
        the caller's array is gathered afterwards"""
        view = getattr(self.lowered, "out_view", None)
        if view is None:
            return out, None
        if self._out_gather is None:
            g = ops.Gather(view.shape, view.tables, _TORCH_DTYPE[view.dtype], out.numel(), out.device)
            self._out_gather = (g, torch.empty(out.numel(), dtype=g.dtype, device=out.device))
        return self._out_gather[1], self._out_gather[0]

    def _run(self, in0, in1, out, add=None):
        cfg = self.params.to_config() if self.params is not None else None
        k0, k1 = self._kernel_inputs(in0, in1)
        kout, g = self._kernel_output(out)
        ops.run_desc(self.lowered.op_code, self.lowered.desc, k0, k1, kout, config=cfg, add=add)
        if g is not None:
            g(kout, out)

    def __call__(self, *arrays):
        self._run(*self._pick(arrays))

    def time_evaluator(self, func_name=None, ctx=None, number=10, repeat=1, min_repeat_ms=0):
        def evaluator(*arrays):
            picked = self._pick(arrays)
            out = picked[2]
            in0, in1 = self._kernel_inputs(picked[0], picked[1])
            cfg = self.params.to_config() if self.params is not None else None
            kout, og = self._kernel_output(out)
            secs = ops.time_op(self.lowered.op_code, self.lowered.desc, in0, in1, kout, config=cfg,
                               number=number, repeat=repeat, min_repeat_ms=min_repeat_ms,
                               add=picked[3] if len(picked) > 3 else None)
            for k in self._computed_args:   # element-wise stages in front of an operand run on every call
                e, ins, buf = self._computed_operand(k, arrays)
                extra = e.time(ins, buf, number=number, repeat=repeat, min_repeat_ms=min_repeat_ms)
                secs = [a + b for a, b in zip(secs, extra)]
            if og is not None:   # the reordering of the result runs on every call too
                extra = og.time(kout, out, number=number, repeat=repeat, min_repeat_ms=min_repeat_ms)
                secs = [a + b for a, b in zip(secs, extra)]
            # the stages materialised in front of an operand run on every call: their time counts
            for pos, (g, buf) in self._gathers.items():
                extra = g.time(picked[pos].contiguous(), buf, number=number, repeat=repeat, min_repeat_ms=min_repeat_ms)
                secs = [a + b for a, b in zip(secs, extra)]
            return TimeResult(secs)
        return evaluator

    def get_source(self):
        """what was chosen: the kernel instance and its configuration (the kernels are
        hand-written HIP in libamos_mi355x.so, not generated text)"""
        cfg = self.params.to_config() if self.params is not None else None
        name = ops.kernel_name(self.lowered.op_code, self.lowered.desc, cfg)
        return "// %s\n// %s\n// config: %s\n" % (name, self.lowered, self.params)


def build(sch, args, target="hip", target_host=None, name="default_function"):
    """schedule (with a kernel config applied by a ScheduleApplier) -> runnable Module"""
    lowered = getattr(sch, "lowered", None)
    if lowered is None:
        from .lowering import lower_main_op
        from .. import te
        from .hw_abstraction import compute_dag_from_tensors
        dag = compute_dag_from_tensors([op.output(0) for op in sch.outputs])
        mains = [op for op in dag.op_lst if op.reduce_axis]
        if not mains:
            raise ValueError("nothing to build: apply a schedule from auto_tensorize first")
        lowered = lower_main_op(mains[0], dag)
    return Module(lowered, getattr(sch, "kernel_config", None), list(args))
