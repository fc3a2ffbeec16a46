"""Measurement: MeasureOptions and evaluate_params.

Mirrors python/tvm/auto_tensorize/search/measure.py: MeasureOptions (:26-61, same defaults),
evaluate_params (:319-338, returns milliseconds).  The reference builds and runs candidates
in sub-processes with time-outs; here a candidate is an already compiled kernel instance, so
measuring is one amos_time call (time_evaluator semantics) in this process.
"""
import torch

from .schedule import MAX_FLOAT  # noqa: F401


class MeasureOptions(object):
    def __init__(self, target="llvm", build_func="default", target_host="llvm", timeout=10, verbose=1,
                 number=100, repeat=1, min_repeat_ms=150, cooldown_interval=0, enable_cpu_cache_flush=1,
                 dev_id=0, use_rpc=False, key=None, host=None, port=None, priority=1):
        self.target = target
        self.build_func = build_func
        self.target_host = target_host
        self.timeout = timeout
        self.verbose = verbose
        self.number = number
        self.repeat = repeat
        self.min_repeat_ms = min_repeat_ms
        self.cooldown_interval = cooldown_interval
        self.enable_cpu_cache_flush = enable_cpu_cache_flush
        self.dev_id = dev_id
        self.use_rpc = use_rpc
        self.key = key
        self.host = host
        self.port = port
        self.priority = priority


_TORCH_DTYPE = {"float16": torch.float16, "bfloat16": torch.bfloat16, "int8": torch.int8,
                "float32": torch.float32, "int32": torch.int32}


def random_device_arrays(lowered, dev_id=0, seed=0):
    """inputs uniform[-1, 1] (integers: full range), as the reference fills its arrays
    (search/measure.py:95-108); returns (in0, in1, out) torch tensors on the device"""
    if not torch.cuda.is_available():
        raise RuntimeError("measuring needs a GPU: no HIP device is visible")
    dev = torch.device("cuda", dev_id)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    arrays = []
    for t in lowered.inputs:
        shape = [int(s) for s in t.shape]
        if t.dtype == "int8":
            arrays.append(torch.randint(-128, 128, shape, dtype=torch.int8, device=dev, generator=gen))
        else:
            arrays.append((torch.rand(shape, device=dev, generator=gen) * 2 - 1).to(_TORCH_DTYPE[t.dtype]))
    for pos, const in getattr(lowered, "constants", {}).items():
        arrays[pos] = torch.from_numpy(const).to(dev)
    out = torch.empty([int(s) for s in lowered.output.shape], dtype=_TORCH_DTYPE[lowered.output.dtype], device=dev)
    return arrays[0], arrays[1], out


def random_add_array(lowered, dev_id=0, seed=1):
    """the operand of a fused tail (None without one), filled like the inputs"""
    t = getattr(lowered, "add_input", None)
    if t is None:
        return None
    dev = torch.device("cuda", dev_id)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    shape = [int(s) for s in t.shape]
    if t.dtype == "int32":
        return torch.randint(-(1 << 16), 1 << 16, shape, dtype=torch.int32, device=dev, generator=gen)
    return (torch.rand(shape, device=dev, generator=gen) * 2 - 1).to(_TORCH_DTYPE[t.dtype])


def evaluate_params_on_device(lowered, params, measure_opt):
    """milliseconds per launch of one kernel configuration"""
    from .. import ops
    in0, in1, out = random_device_arrays(lowered, measure_opt.dev_id)
    # stages materialised in front of an operand: the same for every configuration, timed once
    extra, ins = 0.0, [in0, in1]
    for pos, view in getattr(lowered, "gathers", {}).items():
        g = ops.Gather(view.shape, view.tables, _TORCH_DTYPE[view.dtype], ins[pos].numel(), ins[pos].device)
        src = ins[pos]
        ins[pos] = g(src)
        if not hasattr(lowered, "_gather_seconds"):
            lowered._gather_seconds = {}
        if pos not in lowered._gather_seconds:
            t = g.time(src, ins[pos], number=measure_opt.number, repeat=1, min_repeat_ms=measure_opt.min_repeat_ms)
            lowered._gather_seconds[pos] = t[0]
        extra += lowered._gather_seconds[pos]
    for pos, stage in getattr(lowered, "computed", {}).items():
        # an element-wise stage in front of an operand: the same for every configuration, timed once
        # on arrays of the right size (ins[pos] stands for its result in the kernel's timing)
        if not hasattr(lowered, "_eltwise_seconds"):
            lowered._eltwise_seconds = {}
        if pos not in lowered._eltwise_seconds:
            src = torch.empty([int(e) for e in stage.tensor.shape], dtype=_TORCH_DTYPE[stage.tensor.dtype],
                              device=out.device).zero_()
            e = ops.Eltwise(stage.program, len(stage.inputs), src.dtype, src.numel())
            lowered._eltwise_seconds[pos] = e.time([src] * len(stage.inputs), torch.empty_like(src),
                                                   number=measure_opt.number, repeat=1,
                                                   min_repeat_ms=measure_opt.min_repeat_ms)[0]
        extra += lowered._eltwise_seconds[pos]
    view = getattr(lowered, "out_view", None)
    if view is not None:   # the result is reordered behind the kernel: the same for every configuration
        if not hasattr(lowered, "_out_gather_seconds"):
            g = ops.Gather(view.shape, view.tables, _TORCH_DTYPE[view.dtype], out.numel(), out.device)
            lowered._out_gather_seconds = g.time(out.reshape(-1).clone(), out, number=measure_opt.number, repeat=1,
                                                 min_repeat_ms=measure_opt.min_repeat_ms)[0]
        extra += lowered._out_gather_seconds
    secs = ops.time_op(lowered.op_code, lowered.desc, ins[0], ins[1], out, config=params.to_config(),
                       number=measure_opt.number, repeat=max(1, measure_opt.repeat),
                       min_repeat_ms=measure_opt.min_repeat_ms, add=random_add_array(lowered, measure_opt.dev_id))
    return (sum(secs) / len(secs) + extra) * 1e3


def evaluate_params(schedule_app, params, measure_opt, timeout=100, dump=False):
    """cost in milliseconds (reference: search/measure.py:319-338); MAX_FLOAT on failure"""
    from .. import _lib
    try:
        if dump:
            print("Kernel:", schedule_app.lowered, params, flush=True)
        return evaluate_params_on_device(schedule_app.lowered, params, measure_opt)
    except (_lib.AmosError, RuntimeError) as e:
        print("Bad params, error message:", flush=True)
        print(e, flush=True)
        return MAX_FLOAT
