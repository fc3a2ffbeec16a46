"""Mappings: which loops of the compute go onto the intrinsic's axes.

Mirrors python/tvm/auto_tensorize/tensorization_phases/compute_transform.py: Record
(:228-243), VMappingGenerator's unified subsets of the match points (:115-207),
MappingGenerator.get_all (:291-295), MappingApplier.apply with its strict feasibility rule
(:343-504).  Enumeration and feasibility run in C++ (amos_enumerate_mappings).  The reference
then rewrites the TE compute into im2col-like stages; here the result of `apply` is a
MappingState that only records the fused loops -- the kernels compute addresses on the fly.
"""
import ctypes
import json

from .. import _lib
from .intrin_match import IntrinMatchResult


class Record(object):
    def __init__(self, vmap_choice):
        self.vmap_choice = vmap_choice        # (bit list, direction)

    def to_json(self):
        return {"vmap": [list(self.vmap_choice[0]), self.vmap_choice[1]]}

    def as_key(self):
        return "(" + ",".join(map(str, self.vmap_choice[0])) + ")"

    def as_tuple(self):
        return tuple(self.vmap_choice[0])

    def __str__(self):
        return json.dumps(self.to_json())


def _points_table(axis_map):
    """axis_map {intrinsic IterVar: [target IterVar per point]} -> (intrinsic axes, target axes
    in first-seen order, points as rows of target-axis ids)"""
    intrin_axes = list(axis_map.keys())
    n_points = 0
    for lst in axis_map.values():
        if n_points:
            assert n_points == len(lst)
        n_points = len(lst)
    target_axes, ids = [], {}
    rows = []
    for p in range(n_points):
        row = []
        for ia in intrin_axes:
            tv = axis_map[ia][p]
            if id(tv) not in ids:
                ids[id(tv)] = len(target_axes)
                target_axes.append(tv)
            row.append(ids[id(tv)])
        rows.append(row)
    return intrin_axes, target_axes, rows


def enumerate_mappings(axis_map):
    """[(bits, feasible)] in the reference's enumeration order"""
    intrin_axes, target_axes, rows = _points_table(axis_map)
    n_points, n_axes = len(rows), len(intrin_axes)
    if n_points == 0:
        return []
    flat = (ctypes.c_int32 * (n_points * n_axes))(*[v for r in rows for v in r])
    text = (ctypes.c_int64 * len(target_axes))(*[int(t.dom.extent) for t in target_axes])
    iext = (ctypes.c_int64 * n_axes)(*[int(a.dom.extent) for a in intrin_axes])
    cap = 1 << min(n_points, 15) if n_points <= 15 else n_points + 2
    bits = (ctypes.c_uint8 * (cap * n_points))()
    feas = (ctypes.c_uint8 * cap)()
    n = _lib.check(_lib.load().amos_enumerate_mappings(n_points, n_axes, flat, text, iext, bits, feas, cap))
    return [([int(bits[m * n_points + i]) for i in range(n_points)], bool(feas[m])) for m in range(n)]


class VMappingGenerator(object):
    def __init__(self, axis_map, unify=True):
        assert unify, "only unified enumeration is provided"
        self._all = enumerate_mappings(axis_map)
        self.vmaps = [bits for bits, _ in self._all]
        print(f"Totally {len(self.vmaps)} different mappings for this matching", flush=True)

    def get_all(self):
        return [(v, -1) for v in self.vmaps]


class MappingGenerator(object):
    def __init__(self, intrin_match_result, eps=1e-1, log_file=None, steps=1, allow_repeat=False,
                 topk=3, verbose_init=True):
        assert isinstance(intrin_match_result, IntrinMatchResult)
        if verbose_init:
            print("Logging to %s..." % (log_file if log_file else "devnull"), flush=True)
        self.record_cls = Record
        self.vmap_gen = VMappingGenerator(intrin_match_result.axis_map)

    def record_from_json(self, obj):
        return Record((list(obj["vmap"][0]), obj["vmap"][1]))

    def get_all(self):
        return [Record(v) for v in self.vmap_gen.get_all()]

    def get(self, policy="random"):
        return self.get_all()[0]


class MappingState(object):
    """What a mapping puts on each intrinsic axis: fused target loops (in first-seen order),
    their fused extent, and the loops left as time loops."""

    def __init__(self, match_result, record, fused, time_loops, need_padding):
        self.match_result = match_result
        self.record = record
        self.fused = fused                # {intrinsic IterVar: [target IterVar]}
        self.time_loops = time_loops
        self.need_padding = need_padding
        self.target_dag = match_result.target_dag
        self.intrin_dag = match_result.intrin_dag
        self.main_op_map = match_result.main_op_map

    def fused_names(self):
        return {ia.var.name: [t.var.name for t in lst] for ia, lst in self.fused.items()}


class MappingApplier(object):
    def __init__(self, intrin_match_result, verbose=False, strict=True):
        assert isinstance(intrin_match_result, IntrinMatchResult)
        self.match_result = intrin_match_result
        self.verbose = verbose
        self.strict = strict

    def apply(self, record, drop_output=False):
        """virtual mapping (fuse the selected loops per intrinsic axis) then the concrete step
        (split by the intrinsic extent); raises RuntimeError for an infeasible mapping under
        strict=True exactly where the reference does (compute_transform.py:457-468)"""
        mr = self.match_result
        bits = list(record.vmap_choice[0])
        main_op = list(mr.main_op_map.values())[0]
        target_axes = list(main_op.axis) + list(main_op.reduce_axis)
        fused, used = {}, set()
        need_padding = False
        for ia, lst in mr.axis_map.items():
            if len(lst) == 0:
                continue
            assert len(lst) == len(bits)
            chosen = []
            for tv, b in zip(lst, bits):
                if b and all(tv is not c for c in chosen):
                    chosen.append(tv)
            fused[ia] = chosen
            for c in chosen:
                used.add(id(c))
        for ia, chosen in fused.items():
            factor = int(ia.dom.extent)
            if factor <= 1:
                continue
            extent = 1
            for c in chosen:
                extent *= int(c.dom.extent)
            if extent < factor and self.strict:
                raise RuntimeError(
                    "\nThis mapping is infeasible because it attempts to split a"
                    f" larger dim of extent {factor} from a smaller dim of extent {extent}.\n")
            if extent < factor:
                need_padding = True
        time_loops = [a for a in target_axes if id(a) not in used]
        state = MappingState(mr, record, fused, time_loops, need_padding)
        if self.verbose:
            print("Mapping", str(record), state.fused_names(), "time loops:",
                  [a.var.name for a in time_loops], flush=True)
        return state
