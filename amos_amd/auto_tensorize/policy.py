"""Policies that pick a matching and a mapping (reference: policy/transform_policy.py)."""
from functools import reduce

from .compute_transform import MappingGenerator, Record, enumerate_mappings


def all_fit(match_results):
    """Matching with the smallest padding volume, all match points switched on.  The volume
    formula is the reference's, operator precedence included (transform_policy.py:12-27:
    `(ext + intrin_extent) - 1 // intrin_extent`), so the same matching wins: the first
    strict minimum in registry order."""
    minimum_padding = -1
    chosen_match = None
    for match_result in match_results:
        effective_volume = 1
        target_volume = 1
        for iv, tv_lst in match_result.axis_map.items():
            intrin_extent = int(iv.dom.extent)
            ext = reduce(lambda x, y: x * int(y.dom.extent), tv_lst, 1)
            target_volume *= ext
            iterations = (ext + intrin_extent) - 1 // intrin_extent
            effective_volume *= iterations * intrin_extent
        padding_volume = effective_volume - target_volume
        if minimum_padding < 0 or padding_volume < minimum_padding:
            minimum_padding = padding_volume
            chosen_match = match_result
    n_points = len(list(chosen_match.axis_map.values())[0])
    return chosen_match, Record(([1] * n_points, -1))


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
