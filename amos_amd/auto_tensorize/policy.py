"""Policies that pick a matching and a mapping (reference: policy/transform_policy.py)."""
from functools import reduce

from .compute_transform import MappingGenerator, Record, enumerate_mappings


def _padding_volume(match_result):
    """padded volume minus real volume of the fused loops, by the reference's own arithmetic
    (transform_policy.py:12-27).  Its tile count reads `(ext + intrin_extent) - 1 // intrin_extent`:
    the division binds first, so an axis counts ext + intrin_extent "tiles" (one fewer where the
    intrinsic extent is 1).  Kept as it is: the README's choice of matching depends on it."""
    padded, real = 1, 1
    for intrin_axis, target_axes in match_result.axis_map.items():
        width = int(intrin_axis.dom.extent)
        ext = 1
        for axis in target_axes:
            ext *= int(axis.dom.extent)
        tiles = ext + width - (1 // width)
        padded *= tiles * width
        real *= ext
    return padded - real


def all_fit(match_results):
    """The matching with the smallest padding volume (the first one on a tie, in registry order),
    with every match point switched on."""
    chosen = min(match_results, key=_padding_volume)
    n_points = len(next(iter(chosen.axis_map.values())))
    return chosen, Record(([1] * n_points, -1))


def first_fit(match_results):
    """first matching with a feasible mapping, in enumeration order (the reference shuffles
    the candidates; a deterministic order is used here)"""
    last = None
    for match_result in match_results:
        for bits, feasible in enumerate_mappings(match_result.axis_map):
            last = (match_result, Record((bits, -1)))
            if feasible:
                return last
    assert last is not None
    return last


def default_score_func(value_map):
    total_volume, org_volume = 1, 1
    for k, lst in value_map.items():
        ext = reduce(lambda x, y: x * int(y.dom.extent), lst, 1)
        intrin_extent = int(k.dom.extent)
        tiles = (ext + intrin_extent - 1) / intrin_extent
        total_volume *= tiles * intrin_extent
        org_volume *= ext
    return (total_volume - org_volume) / (org_volume + 1e-5)


def best_fit(match_results, score_func=default_score_func):
    """matching and mapping with the smallest relative padding (transform_policy.py:86-131)"""
    best = None
    for match_result in match_results:
        for bits, _ in enumerate_mappings(match_result.axis_map):
            value = {}
            for k, lst in match_result.axis_map.items():
                uniq = []
                for tv, b in zip(lst, bits):
                    if b and all(tv is not u for u in uniq):
                        uniq.append(tv)
                value[k] = uniq
            score = score_func(value)
            if best is None or score < best[2]:
                best = (match_result, bits, score)
    assert best is not None
    return best[0], Record((best[1], -1))


def choose_one(match_results, match_id, mapping_id):
    assert match_id < len(match_results)
    match_result = match_results[match_id]
    mappings = MappingGenerator(match_result).get_all()
    print("List all possible mappings for this matching", flush=True)
    for i, m in enumerate(mappings):
        print(i, ":", str(m), flush=True)
    assert mapping_id < len(mappings)
    return match_result, mappings[mapping_id]
