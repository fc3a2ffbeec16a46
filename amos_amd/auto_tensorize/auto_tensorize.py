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


def auto_tensorize_v4(target_dag, target, schedule_log_file, measure_opt, schedule_log_dir="schedules",
                      trials=200, repeat_rounds=10, builder=None, runner=None, verbose_schedule=False,
                      transform_dump=False, transform_strict=True, search_group_size=5,
                      desired_compute_key=None, desired_shape_key=None, enable_split_K=False,
                      use_shared_store=False, drop_output=False, build_parallel=1, run_parallel=1,
                      explore_full_match=False, enable_perf_model=False, perf_percentage=0.5):
    """explore every feasible mapping, re-weighting the trial budget between rounds by a
    softmax with momentum over each mapping's best value (auto_tensorize.py:784-811,1018-1035)"""
    measure_opt.target = target
    _check_target(target)
    match_results = get_match_results(target_dag, target)
    if len(match_results) == 0:
        print("This workload has no matched intrinsic for target: %s" % target, flush=True)
        return AutoTensorizeResult()
    print("Possible matchings:", flush=True)
    for i, m in enumerate(match_results):
        print(i, ":", str(m), flush=True)
    if desired_compute_key is not None:
        match_results = [m for m in match_results if m.compute_key == desired_compute_key]
        if not match_results:
            print("No match result matches desired compute key:", desired_compute_key, flush=True)
            return AutoTensorizeResult()
    if desired_shape_key is not None:
        match_results = [m for m in match_results if m.shape_key == desired_shape_key]
        if not match_results:
            print("No match result matches desired shape key:", desired_shape_key, flush=True)
            return AutoTensorizeResult()
    if not explore_full_match:
        match_result, _ = all_fit(match_results)
        match_results = [match_result]

    all_matches, all_mappings, appliers, mapping_weights, weights_updates = [], [], [], [], []
    momentum = 0.8
    total_mappings = 0
    for match_result in match_results:
        mappings = MappingGenerator(match_result).get_all()
        feasible = []
        tmp_app = MappingApplier(match_result, strict=transform_strict)
        for mapping in mappings:
            try:
                tmp_app.apply(mapping, drop_output=drop_output)
                feasible.append(mapping)
            except RuntimeError:
                print("Catch an infeasible mapping:", flush=True)
                print(mapping, flush=True)
        if not feasible:
            continue
        all_matches.append(match_result)
        all_mappings.append(feasible)
        total_mappings += len(feasible)
        mapping_weights.append([1.0 / len(feasible) for _ in feasible])
        weights_updates.append([0.0 for _ in feasible])
        appliers.append(MappingApplier(match_result, verbose=transform_dump, strict=transform_strict))
    total_matchings = len(all_matches)
    if total_mappings == 0:
        print("Can't find any mappings!", flush=True)
        return AutoTensorizeResult()

    pure_test = False
    if trials == 0:
        pure_test = True
        repeat_rounds = 1
        print("Pure testing mode...", flush=True)
    elif trials < total_mappings * repeat_rounds * search_group_size:
        need = total_mappings * repeat_rounds * search_group_size
        print(f"[Warning] Too few trials, expect at least {need} trials.", flush=True)
        trials = need
        print(f"Increase trials to {need}.", flush=True)
    else:
        print("Total trials:", trials, flush=True)
    trials_per_matching = trials // repeat_rounds // total_matchings
    print("Num rounds:", repeat_rounds, flush=True)
    print("Num matching:", total_matchings, flush=True)
    print("Num mapping:", total_mappings, flush=True)
    print("Initial trials per matching:", trials_per_matching, flush=True)
    if not (os.path.exists(schedule_log_dir) and os.path.isdir(schedule_log_dir)):
        os.mkdir(schedule_log_dir)

    class ScheduleContext:
        def __init__(self, schedule_gen, schedule_app, pipeline):
            self.schedule_gen, self.schedule_app, self.pipeline = schedule_gen, schedule_app, pipeline

    cache = {}
    runnable_total = 0
    best_value, best_ctx, best_params, best_mapping = 1 / MAX_FLOAT, None, None, None
    checker = MI355XProgramChecker(verbose_init=False)
    beg = time.time()
    for rnd in range(repeat_rounds):
        for match_id in range(total_matchings):
            match_result, app = all_matches[match_id], appliers[match_id]
            weights, updates = mapping_weights[match_id], weights_updates[match_id]
            tune_trials = [math.ceil(trials_per_matching * x) for x in weights]
            best_values = []
            print("Original weights", weights, flush=True)
            print("Original trials for each mapping", tune_trials, flush=True)
            print("Current explored matching:", str(match_result), flush=True)
            print("Its axis mapping:", flush=True)
            for i, v in match_result.axis_map.items():
                print(i.var, ":", [x.var for x in v], flush=True)
            # the mappings the kernel family realises: pipeline -> bit vector
            realised = {}
            for pipe in (_lib.AMOS_PIPE_PATCH, _lib.AMOS_PIPE_STAGED):
                realised.setdefault(tuple(mapping_of_pipeline(match_result, pipe)), pipe)
            if rnd == 0:
                # trials only for mappings that can run: the others keep weight 0
                runnable = [_realisation(match_result, r, realised) is not None for r in all_mappings[match_id]]
                print("Num runnable mapping:", sum(runnable), flush=True)
                runnable_total += sum(runnable)
                if any(runnable):
                    weights = [w if ok else 0.0 for w, ok in zip(weights, runnable)]
                    total = sum(weights)
                    weights = [w / total for w in weights]
                    mapping_weights[match_id] = weights
                    tune_trials = [math.ceil(trials_per_matching * x) for x in weights]
                    print("Weights of the runnable mappings", weights, flush=True)
            for mapping_id, record in enumerate(all_mappings[match_id]):
                print("Current explored mapping:", str(record), flush=True)
                new_state = app.apply(record, drop_output=drop_output)
                key = record.as_key()
                log = os.path.join(schedule_log_dir, "mapping_" + str(key) + "_" + schedule_log_file)
                value, params = 1 / MAX_FLOAT, None
                how = _realisation(match_result, record, realised)
                if how is None:
                    print("No kernel instance realises this mapping; skipped.", flush=True)
                else:
                    pipes, rows = how
                    if key not in cache:
                        try:
                            gen = MI355XScheduleGenerator(
                                match_result, new_state, log_file=log, rows=rows,
                                perf_percentage=perf_percentage if enable_perf_model else 1.0)
                        except NoKernelError as e:
                            print("No kernel for this compute:", e, flush=True)
                            gen = None
                        if gen is not None:
                            if os.path.exists(log) and os.path.getsize(log) > 0:
                                gen.load_from_file(log)
                            gen._candidates = gen.candidates(pipes)
                            cache[key] = ScheduleContext(gen, MI355XScheduleApplier(match_result, gen.lowered), pipes[0])
                    ctx = cache.get(key)
                    if ctx is not None:
                        if tune_trials[mapping_id] and not pure_test:
                            find_optimized_parameters(match_result, ctx.schedule_gen, ctx.schedule_app,
                                                      measure_opt, checker, tune_trials[mapping_id],
                                                      verbose=verbose_schedule)
                        if ctx.schedule_gen.has_entry():
                            entry = ctx.schedule_gen.get_best_entry()
                            params, value = entry.record, entry.value
                        elif pure_test and ctx.schedule_gen.candidates():
                            params = ctx.schedule_gen.candidates()[0]
                            value = 1.0 / ctx.schedule_gen.estimate(params)
                        if value > best_value:
                            best_value, best_ctx, best_params, best_mapping = value, ctx, params, record
                best_values.append(value)
                print(f"Best record value:{best_value} (larger is better)", flush=True)
                print(f"Round {rnd+1}, Match {match_id+1}, Mapping {mapping_id+1}: {value}/{best_value}"
                      f"({1/best_value*1e3} ms), {str(record)}, {str(params)}", flush=True)
            if not pure_test:
                # (mappings without a kernel stay at weight 0: the update is over the runnable ones)
                ran = [v > 1 / MAX_FLOAT for v in best_values]
                max_value = max(best_values)
                exp_scores = [math.exp(min(0.0, x - max_value)) for x in best_values]
                s = sum(exp_scores)
                new_weights = [x / s for x in exp_scores]
                delta = [new_weights[i] - weights[i] for i in range(len(weights))]
                new_updates = [delta[i] + momentum * updates[i] for i in range(len(updates))]
                new_weights = [weights[i] + new_updates[i] for i in range(len(new_updates))]
                exp_scores = [math.exp(x) if ok or not any(ran) else 0.0 for x, ok in zip(new_weights, ran)]
                s = sum(exp_scores)
                mapping_weights[match_id] = [x / s for x in exp_scores]
                weights_updates[match_id] = new_updates
                print("New weights", mapping_weights[match_id], flush=True)
        if not pure_test:
            print("Show mapping exploration summary:", flush=True)
            for k, v in cache.items():
                print(f"mapping {str(k)}: explored {v.schedule_gen.num_entries()} schedules", flush=True)
    if not pure_test:
        print(f"Mapping exploration uses time {(time.time() - beg)} s.", flush=True)
    result = AutoTensorizeResult() if best_ctx is None else AutoTensorizeResult(
        best_ctx.schedule_gen, best_ctx.schedule_app, best_params, 1 / best_value, mapping=best_mapping)
    result.num_runnable_mappings, result.num_feasible_mappings = runnable_total, total_mappings
    return result


def _realisation(match_result, record, realised):
    """How a mapping runs: (pipelines, rows) or None.  `rows` names the output loops fused into the
    rows of the implicit GEMM where that is not all of them (lowering.remap_conv2d_rows: a 2-d
    convolution whose mapping keeps the batch loop and leaves p and / or q as time loops); the
    reduce side decides the kernel -- channels only: the patch-staged kernels, whose window taps
    are time loops; channels and both window loops: the register-staged kernel (im2col)."""
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
