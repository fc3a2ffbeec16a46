"""Schedule parameters, their generator / applier, the resource checker and the parameter
search for the MI355X kernels.

In the reference a schedule is a set of TE tiling factors (CUDAParamsV2: inline, vectorize,
spatial_factors, reduce_factors, ...; schedulers/cuda_v2.py:42-52) found by simulated
annealing over compile-and-measure trials (search/parameter.py:152-459).  Here a schedule is
a kernel configuration -- block tile, split of the reduction, pipeline -- and the search is
a sweep over the compiled instances that pass the resource check, each timed on the GPU.
The log keeps the reference's JSON-lines shape {"record": ..., "value": 1/seconds}
(search/parameter.py:269-278, search/record.py:1-11) so load_from_file / get_best_entry
scripts keep working.
"""
import ctypes
import heapq
import json
import os

from .. import _lib
from .lowering import lower_main_op

MAX_FLOAT = 1e10


class KernelParams(object):
    """record of one schedule: the fields of amos_kernel_config_t"""

    def __init__(self, tile_i=0, tile_j=0, split_k=1, pipeline=0):
        self.tile_i, self.tile_j, self.split_k, self.pipeline = int(tile_i), int(tile_j), int(split_k), int(pipeline)

    def to_json(self):
        return {"tile_i": self.tile_i, "tile_j": self.tile_j, "split_k": self.split_k, "pipeline": self.pipeline}

    @classmethod
    def from_json(cls, obj):
        return cls(obj["tile_i"], obj["tile_j"], obj.get("split_k", 1), obj.get("pipeline", 0))

    def to_config(self):
        c = _lib.KernelConfig()
        c.tile_i, c.tile_j, c.split_k, c.pipeline = self.tile_i, self.tile_j, self.split_k, self.pipeline
        return c

    def __str__(self):
        return json.dumps(self.to_json())


class Entry(object):
    def __init__(self, record, value):
        self.record = record
        self.value = value

    def __lt__(self, other):
        return self.value > other.value      # max-heap on value = 1/seconds

    def to_json(self):
        return {"record": self.record.to_json(), "value": self.value}


def read_log(file_name):
    """a tuning log as [(record dict, value)]: one JSON object {"record": ..., "value": 1/seconds}
    per line (reference: search/parameter.py:269-278, :294-316)"""
    out = []
    with open(file_name, "r") as fin:
        for line in fin:
            line = line.strip()
            if line:
                obj = json.loads(line)
                out.append((obj["record"], obj["value"]))
    return out


class CheckError(Exception):
    pass


class MI355XProgramChecker(object):
    """LDS bytes and accumulator registers of a config against the gfx950 budget
    (reference: search/checker.py:43-82 with src/auto_tensorize/utils.cc:31-57)"""

    def __init__(self, arch="gfx950", verbose_init=True):
        if verbose_init:
            print("Using arch: %s" % arch, flush=True)

    def check(self, lowered, params):
        lds, regs = ctypes.c_int64(), ctypes.c_int64()
        cfg = params.to_config()
        rc = _lib.load().amos_check_config(lowered.op_code, ctypes.byref(lowered.desc), ctypes.byref(cfg),
                                           ctypes.byref(lds), ctypes.byref(regs))
        if rc < 0:
            raise CheckError(_lib.load().amos_last_error().decode())
        return lds.value, regs.value


class EmptyChecker(object):
    def check(self, lowered, params):
        return 0, 0


_TILES = [(256, 256), (256, 128), (128, 256), (128, 128), (256, 64), (64, 256), (128, 64), (64, 128), (64, 64)]

# which reference-style mapping a pipeline realises for a convolution: the patch-staged kernel
# keeps the window taps as time loops (rk = channels only), the register-staged kernel fuses
# channels and taps into rk (im2col)
def mapping_of_pipeline(match_result, pipeline):
    names = {ia.var.name: [t.var.name for t in lst] for ia, lst in match_result.axis_map.items()}
    rk_key = [k for k in names if k.startswith("r")][0]
    n_points = len(names[rk_key])
    if pipeline in (_lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8):
        first = names[rk_key][0]      # the channel axis sorts first among reduce axes (rc < rd < rr < rs)
        return [1 if names[rk_key][p] == first else 0 for p in range(n_points)]
    return [1] * n_points


class MI355XScheduleGenerator(object):
    def __init__(self, intrin_match_result, new_state=None, log_file="mi355x_schedule_generator.log",
                 arch="gfx950", verbose_init=True, **kwargs):
        self.match_result = intrin_match_result
        self.state = new_state
        main_op = list(intrin_match_result.main_op_map.values())[0]
        self.lowered = lower_main_op(main_op, getattr(intrin_match_result, "target_dag", None))
        # a mapping that fuses only some of the output loops into the rows of the implicit GEMM
        rows = kwargs.get("rows")
        if rows is not None:
            from .lowering import remap_conv2d_rows
            self.lowered = remap_conv2d_rows(self.lowered, rows)
        self.log_file = log_file
        self.verbose_init = verbose_init
        self.entries = []
        self.visited = {}
        self._open_log()
        self._candidates = None
        self._cursor = 0
        # fraction of the model-ranked candidates the sweep may measure (1.0 = all)
        self.perf_percentage = float(kwargs.get("perf_percentage", 1.0))

    # ---- log ------------------------------------------------------------------------------
    def _open_log(self):
        if self.log_file:
            if self.verbose_init:
                print("Logging to %s..." % self.log_file, flush=True)
            self.logger = open(self.log_file, "a")
        else:
            if self.verbose_init:
                print("Logging to %s..." % "devnull", flush=True)
            self.logger = open(os.devnull, "w")

    def record_from_json(self, obj):
        return KernelParams.from_json(obj)

    def feedback(self, record, value, log_to_file=True):
        entry = Entry(record, value)
        self.visited[str(record)] = value
        heapq.heappush(self.entries, entry)
        if log_to_file:
            print(json.dumps(entry.to_json()), file=self.logger, flush=True)

    def clear(self, log_file):
        self.entries, self.visited = [], {}
        self._cursor = 0
        self.log_file = log_file
        self.logger.close()
        self._open_log()

    def load_from_file(self, file_name, clear=False):
        if clear:
            print("Clearing...")
            self.clear(file_name)
        if self.verbose_init:
            print("Loading from file %s..." % file_name, flush=True)
        assert not self.entries, "Please clear the generator first (be caution!)."
        count, best = 0, 0.0
        for record, value in read_log(file_name):
            count += 1
            best = max(value, best)
            self.feedback(self.record_from_json(record), value, False)
        if self.verbose_init:
            print("Load %d entries! The best known is %f ms" % (count, 1 / (best + 1e-10) * 1e3), flush=True)

    def has_entry(self): return len(self.entries) > 0
    def num_entries(self): return len(self.entries)

    def get_best_entry(self):
        assert self.entries
        return self.entries[0]

    def topk(self, k=1):
        return heapq.nsmallest(min(k, len(self.entries)), self.entries)

    # ---- candidates -------------------------------------------------------------------------
    def get_schedule_compute_info(self):
        return self.lowered

    def candidates(self, pipelines=None):
        """configs with a kernel instance that pass the resource check, the mapper's own choice first"""
        if self._candidates is not None and pipelines is None:
            return self._candidates
        lib = _lib.load()
        low = self.lowered
        out, seen = [], set()

        def add(p):
            key = str(p)
            if key in seen:
                return
            cfg = p.to_config()
            if lib.amos_check_config(low.op_code, ctypes.byref(low.desc), ctypes.byref(cfg), None, None) < 0:
                return
            name = lib.amos_kernel_name(low.op_code, ctypes.byref(low.desc), ctypes.byref(cfg))
            if name is None:
                return
            # two pipelines may resolve to one kernel (a pointwise convolution runs as a matrix
            # product whatever is asked for short of the patch pipelines): time it once
            launch = (name, p.tile_i, p.tile_j, p.split_k)
            if launch in seen:
                return
            seen.add(key)
            seen.add(launch)
            out.append(p)

        d = _lib.KernelConfig()
        if lib.amos_default_config(low.op_code, ctypes.byref(low.desc), ctypes.byref(d)) == 0 and (
                pipelines is None or d.pipeline in pipelines):
            add(KernelParams(d.tile_i, d.tile_j, d.split_k, d.pipeline))
        is_conv = low.kind in ("conv2d", "conv3d")
        pipes = pipelines if pipelines is not None else (
            [_lib.AMOS_PIPE_NCHW, _lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8, _lib.AMOS_PIPE_STAGED, _lib.AMOS_PIPE_AUTO] if is_conv
            else [_lib.AMOS_PIPE_AUTO, _lib.AMOS_PIPE_STAGED])
        first = len(out)
        for pipe in pipes:
            for ti, tj in _TILES:
                for split in (1, 2, 4, 8):
                    if split > 1 and low.kind == "bgemm":
                        continue
                    add(KernelParams(ti, tj, split, pipe))
        # The sweep visits candidates in the order of the analytical model (the mapper's own
        # choice stays first), so that a small trial budget is spent on the likely winners; the
        # reference ranks candidates with its performance model the same way before measuring
        # (auto_tensorize.py:1018-1035, backend/tenet_integrate.py:168-202).
        out[first:] = sorted(out[first:], key=self.estimate)
        if self.perf_percentage < 1.0:
            keep = max(1, int(round(len(out) * self.perf_percentage)))
            out = out[:keep]
        if pipelines is None:
            self._candidates = out
        return out

    def get_next(self, policy="sweep"):
        cands = self.candidates()
        while self._cursor < len(cands):
            p = cands[self._cursor]
            self._cursor += 1
            if str(p) not in self.visited:
                return p
        return None

    def estimate(self, params):
        sec = ctypes.c_double()
        cfg = params.to_config()
        rc = _lib.load().amos_estimate_seconds(self.lowered.op_code, ctypes.byref(self.lowered.desc),
                                               ctypes.byref(cfg), ctypes.byref(sec))
        if rc != 0:
            return MAX_FLOAT
        # stages materialised around the kernel (gathers of an operand, of the result): a launch
        # each, their bytes read and written once at about a quarter of the HBM rate
        extra = 0.0
        views = list(self.lowered.gathers.values()) + ([self.lowered.out_view] if self.lowered.out_view is not None else [])
        for v in views:
            n = 1
            for e in v.shape:
                n *= int(e)
            width = {"float16": 2, "bfloat16": 2, "int8": 1}.get(v.dtype, 4)
            extra += 3e-6 + 2.0 * n * width / 2.0e12
        return sec.value + extra


class MI355XScheduleApplier(object):
    def __init__(self, intrin_match_result, schedule_compute_info):
        self.match_result = intrin_match_result
        self.lowered = schedule_compute_info
        self.target_dag = intrin_match_result.target_dag

    def apply(self, sch, params, mapping_func=lambda x: [x]):
        sch.kernel_config = params
        sch.lowered = self.lowered
        return sch


def find_optimized_parameters(match_results, schedule_gen, schedule_app, measure_opt, checker, trials,
                              search_group_size=16, policy="", builder=None, runner=None, verbose=False,
                              build_parallel=1, run_parallel=1):
    """time up to `trials` unvisited candidates, log each, return (best value, best params)
    (reference: search/parameter.py:386-459; value = 1/seconds)"""
    from .measure import evaluate_params_on_device
    best_value, best_params = 1 / MAX_FLOAT, None
    if schedule_gen.has_entry():
        top = schedule_gen.get_best_entry()
        best_value, best_params = top.value, top.record
    done = 0
    while done < trials:
        params = schedule_gen.get_next()
        if params is None:
            break
        done += 1
        try:
            checker.check(schedule_gen.lowered, params)
            ms = evaluate_params_on_device(schedule_app.lowered, params, measure_opt)
            value = 1.0 / (ms * 1e-3)
            print(".Y*Y", end="", flush=True)
        except (CheckError, _lib.AmosError) as e:
            value = 1 / MAX_FLOAT
            print(".E", end="", flush=True)
            if verbose:
                print("\n", e, flush=True)
        schedule_gen.feedback(params, value)
        if value > best_value:
            best_value, best_params = value, params
    print(flush=True)
    if done:
        print("iteration=1: %s/%s" % (best_value, best_value), flush=True)
    return best_value, best_params
