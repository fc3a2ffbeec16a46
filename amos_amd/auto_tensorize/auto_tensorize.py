"""The API driver: auto_tensorize, auto_tensorize_v4, AutoTensorizeResult, get_schedule.

Mirrors python/tvm/auto_tensorize/auto_tensorize.py (:37-51 result type, :54-114 compute
mapping, :117-239 schedule search, :242-291 auto_tensorize, :294-301 get_schedule,
:661-1053 auto_tensorize_v4) including its console protocol, with the CUDA schedule
generators replaced by the MI355X kernel-configuration sweep.
"""
import math
import os
import time

from .. import te
from .compute_transform import MappingApplier, MappingGenerator
from .intrin_match import get_match_results
from .lowering import NoKernelError
from .policy import all_fit, best_fit, choose_one, first_fit
from .schedule import (MAX_FLOAT, EmptyChecker, KernelParams, MI355XProgramChecker,
                       MI355XScheduleApplier, MI355XScheduleGenerator, find_optimized_parameters,
                       mapping_of_pipeline)
from .. import _lib

_TARGETS = ("hip", "rocm")


class AutoTensorizeResult(object):
    def __init__(self, sch_gen=None, sch_app=None, params=None, perf=None, mapping=None):
        self.sch_gen = sch_gen
        self.sch_app = sch_app
        self.params = params
        self.perf = perf          # seconds per run
        self.mapping = mapping
        # auto_tensorize_v4: how many of the feasible mappings a kernel could run, and how many there were
        self.num_runnable_mappings = None
        self.num_feasible_mappings = None

    def defined(self):
        return ((self.sch_gen is not None) and (self.sch_app is not None)
                and (self.params is not None) and (self.perf is not None))


def _check_target(target):
    if str(target) not in _TARGETS:
        raise RuntimeError("Do not support target: %s (this build targets %s)" % (target, " / ".join(_TARGETS)))


def auto_tensorize_compute(target_dag, target, log_file, measure_opt, verbose=False, transform_dump=False,
                           transform_strict=True, drop_output=False, transform_policy="all_fit"):
    measure_opt.target = target
    _check_target(target)
    match_results = get_match_results(target_dag, target)
    if len(match_results) == 0:
        print("This workload has no matched intrinsic for target: %s" % target, flush=True)
        return None, None
    print("Possible matchings:", flush=True)
    for i, m in enumerate(match_results):
        print(i, ":", str(m), flush=True)
    if transform_policy == "all_fit":
        match_result, record = all_fit(match_results)
    elif transform_policy == "first_fit":
        match_result, record = first_fit(match_results)
    elif transform_policy == "best_fit":
        match_result, record = best_fit(match_results)
    elif transform_policy[:7] == "choose:":
        mat_id, map_id = transform_policy[7:].split(",")
        match_result, record = choose_one(match_results, int(mat_id), int(map_id))
    else:
        raise RuntimeError("Unknown transform policy: %s" % transform_policy)
    print("Selected matching:", str(match_result), flush=True)
    print("Axis mapping:", flush=True)
    for i, v in match_result.axis_map.items():
        print(i.var, ":", [x.var for x in v], flush=True)
    print("Selected mapping:", str(record), flush=True)
    if getattr(match_result.hw_abs_dag, "wrapped_spelling", False):
        print("[Warning] int8 product spelled (a * b).astype(\"int32\"): an llvm build wraps it to int8, "
              "the matrix core computes exact int32 products", flush=True)
    app = MappingApplier(match_result, verbose=transform_dump, strict=transform_strict)
    new_state = app.apply(record, drop_output=drop_output)
    return match_result, new_state


def auto_tensorize_schedule(target_dag, target, log_file, measure_opt, match_result, new_state, trials=200,
                            builder=None, runner=None, verbose=False, search_group_size=16,
                            enable_split_K=False, use_lagacy=False, build_parallel=1, run_parallel=1):
    if match_result is None or new_state is None:
        return AutoTensorizeResult(None, None, None, None)
    _check_target(target)
    try:
        schedule_gen = MI355XScheduleGenerator(match_result, new_state, log_file=log_file)
    except NoKernelError as e:
        print("No kernel for this compute:", e, flush=True)
        return AutoTensorizeResult(None, None, None, None)
    if log_file and os.path.exists(log_file) and os.path.isfile(log_file) and os.path.getsize(log_file) > 0:
        schedule_gen.load_from_file(log_file)
    sc_info = schedule_gen.get_schedule_compute_info()
    schedule_app = MI355XScheduleApplier(match_result, sc_info)
    checker = MI355XProgramChecker()
    if trials:
        find_optimized_parameters(match_result, schedule_gen, schedule_app, measure_opt, checker, trials,
                                  verbose=verbose, search_group_size=search_group_size)
    if not schedule_gen.has_entry():
        # no measurement (trials=0, empty log): the mapper's analytical choice and estimate
        params = schedule_gen.candidates()[0]
        return AutoTensorizeResult(schedule_gen, schedule_app, params, schedule_gen.estimate(params))
    entry = schedule_gen.get_best_entry()
    return AutoTensorizeResult(schedule_gen, schedule_app, entry.record, 1 / entry.value)


def auto_tensorize(target_dag, target, log_file, measure_opt, trials=200, builder=None, runner=None,
                   verbose=False, transform_dump=False, transform_strict=True, drop_output=False,
                   transform_policy="all_fit", search_group_size=16, enable_split_K=False,
                   build_parallel=1, run_parallel=1):
    print("[AMOS] Mapping starts...\nUsing deterministic mapping logic with dynamic schedule tuning", flush=True)
    match_result, new_state = auto_tensorize_compute(target_dag, target, log_file, measure_opt, verbose,
                                                     transform_dump, transform_strict, drop_output,
                                                     transform_policy)
    return auto_tensorize_schedule(target_dag, target, log_file, measure_opt, match_result, new_state, trials,
                                   builder, runner, verbose, search_group_size, enable_split_K,
                                   build_parallel=build_parallel, run_parallel=run_parallel)


def get_schedule(sch_app, params):
    target_dag = sch_app.target_dag
    inputs = target_dag.get_inputs()
    sch = te.create_schedule([x.op for x in target_dag.tensors])
    args = inputs + list(target_dag.tensors)
    sch = sch_app.apply(sch, params)
    return sch, args


class _TrialShares:
    """How one matching's trial budget is divided between its mappings: a softmax over each
    mapping's best value, moved towards with momentum between rounds (the rule of
    auto_tensorize.py:784-811 and :1018-1035).  Mappings no kernel can run hold a share of 0."""
    MOMENTUM = 0.8

    def __init__(self, count):
        self.shares = [1.0 / count] * count
        self.velocity = [0.0] * count

    def restrict(self, allowed):
        """shares only for the mappings flagged in `allowed` (unless none is)"""
        if any(allowed):
            kept = [w if ok else 0.0 for w, ok in zip(self.shares, allowed)]
            total = sum(kept)
            self.shares = [w / total for w in kept]

    def trials(self, budget):
        return [math.ceil(budget * w) for w in self.shares]

    def update(self, values):
        """one round's best values (1 / MAX_FLOAT = did not run) -> new shares"""
        ran = [v > 1 / MAX_FLOAT for v in values]
        top = max(values)
        target = _normalised([math.exp(min(0.0, v - top)) for v in values])
        self.velocity = [t - w + self.MOMENTUM * u for t, w, u in zip(target, self.shares, self.velocity)]
        moved = [w + u for w, u in zip(self.shares, self.velocity)]
        self.shares = _normalised([math.exp(x) if ok or not any(ran) else 0.0 for x, ok in zip(moved, ran)])


def _normalised(xs):
    total = sum(xs)
    return [x / total for x in xs]


class _MappingRun:
    """the kernel-configuration sweep of one mapping: generator, applier, first pipeline"""

    def __init__(self, schedule_gen, schedule_app, pipeline):
        self.schedule_gen, self.schedule_app, self.pipeline = schedule_gen, schedule_app, pipeline


class _MatchingSweep:
    """one matching of auto_tensorize_v4: its feasible mappings, their trial shares, and which
    of them a kernel family can run"""

    def __init__(self, match_result, transform_strict, transform_dump, drop_output):
        self.match_result = match_result
        self.drop_output = drop_output
        probe = MappingApplier(match_result, strict=transform_strict)
        self.mappings = []
        for mapping in MappingGenerator(match_result).get_all():
            try:
                probe.apply(mapping, drop_output=drop_output)
                self.mappings.append(mapping)
            except RuntimeError:
                print("Catch an infeasible mapping:", flush=True)
                print(mapping, flush=True)
        self.applier = MappingApplier(match_result, verbose=transform_dump, strict=transform_strict)
        self.shares = _TrialShares(len(self.mappings)) if self.mappings else None
        # the mappings the kernel families implement as they are: bit vector -> pipeline
        self.realised = {}
        for pipe in (_lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_STAGED):
            self.realised.setdefault(tuple(mapping_of_pipeline(match_result, pipe)), pipe)

    def how(self, record):
        return _realisation(self.match_result, record, self.realised)

    def announce(self, budget):
        print("Original weights", self.shares.shares, flush=True)
        print("Original trials for each mapping", self.shares.trials(budget), flush=True)
        print("Current explored matching:", str(self.match_result), flush=True)
        print("Its axis mapping:", flush=True)
        for i, v in self.match_result.axis_map.items():
            print(i.var, ":", [x.var for x in v], flush=True)

    def keep_runnable(self):
        """first round: trials only for mappings that can run; returns how many can"""
        runnable = [self.how(r) is not None for r in self.mappings]
        print("Num runnable mapping:", sum(runnable), flush=True)
        if any(runnable):
            self.shares.restrict(runnable)
            print("Weights of the runnable mappings", self.shares.shares, flush=True)
        return sum(runnable)


def auto_tensorize_v4(target_dag, target, schedule_log_file, measure_opt, schedule_log_dir="schedules",
                      trials=200, repeat_rounds=10, builder=None, runner=None, verbose_schedule=False,
                      transform_dump=False, transform_strict=True, search_group_size=5,
                      desired_compute_key=None, desired_shape_key=None, enable_split_K=False,
                      use_shared_store=False, drop_output=False, build_parallel=1, run_parallel=1,
                      explore_full_match=False, enable_perf_model=False, perf_percentage=0.5):
    """Explores every feasible mapping of the chosen matching(s): per round each mapping gets its
    share of the trials (`_TrialShares`) for the kernel-configuration sweep of the kernel family
    that can run it.  Signature and console protocol of the reference's auto_tensorize_v4
    (python/tvm/auto_tensorize/auto_tensorize.py:661-1053)."""
    measure_opt.target = target
    _check_target(target)
    match_results = get_match_results(target_dag, target)
    if len(match_results) == 0:
        print("This workload has no matched intrinsic for target: %s" % target, flush=True)
        return AutoTensorizeResult()
    print("Possible matchings:", flush=True)
    for i, m in enumerate(match_results):
        print(i, ":", str(m), flush=True)
    for wanted, attr, what in ((desired_compute_key, "compute_key", "compute"), (desired_shape_key, "shape_key", "shape")):
        if wanted is None:
            continue
        match_results = [m for m in match_results if getattr(m, attr) == wanted]
        if not match_results:
            print("No match result matches desired %s key:" % what, wanted, flush=True)
            return AutoTensorizeResult()
    if not explore_full_match:
        match_results = [all_fit(match_results)[0]]

    sweeps = [sw for sw in (_MatchingSweep(m, transform_strict, transform_dump, drop_output) for m in match_results)
              if sw.mappings]
    total_mappings = sum(len(sw.mappings) for sw in sweeps)
    if total_mappings == 0:
        print("Can't find any mappings!", flush=True)
        return AutoTensorizeResult()

    pure_test = trials == 0
    if pure_test:
        repeat_rounds = 1
        print("Pure testing mode...", flush=True)
    elif trials < total_mappings * repeat_rounds * search_group_size:
        trials = total_mappings * repeat_rounds * search_group_size
        print(f"[Warning] Too few trials, expect at least {trials} trials.", flush=True)
        print(f"Increase trials to {trials}.", flush=True)
    else:
        print("Total trials:", trials, flush=True)
    budget = trials // repeat_rounds // len(sweeps)
    print("Num rounds:", repeat_rounds, flush=True)
    print("Num matching:", len(sweeps), flush=True)
    print("Num mapping:", total_mappings, flush=True)
    print("Initial trials per matching:", budget, flush=True)
    if not os.path.isdir(schedule_log_dir):
        os.mkdir(schedule_log_dir)

    runs = {}            # mapping key -> _MappingRun (None: no kernel for the compute)
    runnable_total = 0
    best = {"value": 1 / MAX_FLOAT, "run": None, "params": None, "mapping": None}
    checker = MI355XProgramChecker(verbose_init=False)
    started = time.time()

    def run_of(sweep, record, pipes, rows):
        key = record.as_key()
        if key not in runs:
            log = os.path.join(schedule_log_dir, "mapping_" + str(key) + "_" + schedule_log_file)
            try:
                gen = MI355XScheduleGenerator(sweep.match_result, sweep.applier.apply(record, drop_output=drop_output),
                                              log_file=log, rows=rows,
                                              perf_percentage=perf_percentage if enable_perf_model else 1.0)
            except NoKernelError as e:
                print("No kernel for this compute:", e, flush=True)
                runs[key] = None
                return None
            if os.path.exists(log) and os.path.getsize(log) > 0:
                gen.load_from_file(log)
            # a mapping the kernels implement as it is (no remapped loops) is also what the mapper's
            # own choice and its AMOS_PIPE_AUTO resolution run -- the direct-to-LDS GEMM, the
            # depthwise, few-channel and skinny kernels, which have no pipeline value of their own;
            # a remapped one only gets the pipelines of its kernel family
            gen._candidates = gen.candidates(None if rows is None else pipes)
            runs[key] = _MappingRun(gen, MI355XScheduleApplier(sweep.match_result, gen.lowered), pipes[0])
        return runs[key]

    def explore(sweep, record, n_trials):
        """the sweep of one mapping for this round -> (its best value so far, the parameters)"""
        how = sweep.how(record)
        if how is None:
            print("No kernel instance realises this mapping; skipped.", flush=True)
            return 1 / MAX_FLOAT, None
        run = run_of(sweep, record, *how)
        if run is None:
            return 1 / MAX_FLOAT, None
        gen = run.schedule_gen
        if n_trials and not pure_test:
            find_optimized_parameters(sweep.match_result, gen, run.schedule_app, measure_opt, checker, n_trials,
                                      verbose=verbose_schedule)
        value, params = 1 / MAX_FLOAT, None
        if gen.has_entry():
            entry = gen.get_best_entry()
            params, value = entry.record, entry.value
        elif pure_test and gen.candidates():
            params = gen.candidates()[0]
            value = 1.0 / gen.estimate(params)
        if value > best["value"]:
            best.update(value=value, run=run, params=params, mapping=record)
        return value, params

    for rnd in range(repeat_rounds):
        for match_id, sweep in enumerate(sweeps):
            sweep.announce(budget)
            if rnd == 0:
                runnable_total += sweep.keep_runnable()
            per_mapping = sweep.shares.trials(budget)
            values = []
            for mapping_id, record in enumerate(sweep.mappings):
                print("Current explored mapping:", str(record), flush=True)
                value, params = explore(sweep, record, per_mapping[mapping_id])
                values.append(value)
                print(f"Best record value:{best['value']} (larger is better)", flush=True)
                print(f"Round {rnd+1}, Match {match_id+1}, Mapping {mapping_id+1}: {value}/{best['value']}"
                      f"({1/best['value']*1e3} ms), {str(record)}, {str(params)}", flush=True)
            if not pure_test:
                sweep.shares.update(values)
                print("New weights", sweep.shares.shares, flush=True)
        if not pure_test:
            print("Show mapping exploration summary:", flush=True)
            for k, v in runs.items():
                if v is not None:
                    print(f"mapping {str(k)}: explored {v.schedule_gen.num_entries()} schedules", flush=True)
    if not pure_test:
        print(f"Mapping exploration uses time {(time.time() - started)} s.", flush=True)
    run = best["run"]
    result = AutoTensorizeResult() if run is None else AutoTensorizeResult(
        run.schedule_gen, run.schedule_app, best["params"], 1 / best["value"], mapping=best["mapping"])
    result.num_runnable_mappings, result.num_feasible_mappings = runnable_total, total_mappings
    return result


def _realisation(match_result, record, realised):
    """How a mapping runs: (pipelines, rows) or None.  `rows` names the output loops fused into the
    rows of the implicit GEMM where that is not all of them (lowering.remap_conv2d_rows: a 2-d
    convolution whose mapping keeps the batch loop and leaves p and / or q as time loops); the
    reduce side decides the kernel -- channels only: the patch-staged kernels, whose window taps
    are time loops; channels and both window loops: the register-staged kernel (im2col); channels
    and one window loop ("+s" / "+r" behind the rows): the patch-staged kernels on an image whose
    channels hold that loop's taps, the other window loop staying a time loop -- the output loop
    along the folded axis is then a row loop of necessity."""
    patch_family = [_lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_PATCH8, _lib.AMOS_PIPE_NCHW]
    pipe = _equivalent_pipeline(match_result, record, realised)
    if pipe is not None:
        return (patch_family if pipe == _lib.AMOS_PIPE_PATCH else [pipe]), None
    names = {ia.var.name: [t.var.name for t in lst] for ia, lst in match_result.axis_map.items()}
    if sorted(names) != ["i", "j", "rk"]:
        return None
    bits = record.vmap_choice[0]
    i_set = sorted(set(n for n, b in zip(names["i"], bits) if b))
    rk_set = sorted(set(n for n, b in zip(names["rk"], bits) if b))
    spatial, reduce_all = sorted(set(names["i"])), sorted(set(names["rk"]))
    if spatial != ["n", "p", "q"] or reduce_all != ["rc", "rr", "rs"] or "n" not in i_set:
        return None
    if rk_set == ["rc"]:
        # (rows n alone: one image as wide as N*Q*S columns, whose patch of a tile no LDS holds)
        if i_set == ["n"]:
            return None
        pipes = patch_family
    elif rk_set == reduce_all:
        pipes = [_lib.AMOS_PIPE_STAGED]
    elif rk_set == ["rc", "rs"] and "q" in i_set:
        return patch_family, "".join(i_set) + "+s"
    elif rk_set == ["rc", "rr"] and "p" in i_set:
        return patch_family, "".join(i_set) + "+r"
    else:
        return None
    return pipes, "".join(i_set)


def _equivalent_pipeline(match_result, record, realised):
    """a mapping is realised by a pipeline when it puts the same sets of loops on every
    intrinsic axis as the mapping that pipeline implements"""
    def loop_sets(bits):
        return tuple(tuple(sorted(set(t.var.name for t, b in zip(lst, bits) if b)))
                     for lst in match_result.axis_map.values())
    mine = loop_sets(record.vmap_choice[0])
    for bits, pipe in realised.items():
        if loop_sets(bits) == mine:
            return pipe
    return None
