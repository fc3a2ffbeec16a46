"""Writes readme_conv2d_mappings.json: the console facts of the reference's conv2d tutorial
(README.md:203-261 of the reference), typed in from that text.  Nothing of the reference is
imported or run."""
import json
import os

fixture = {
    "source": "README.md:203-261",
    "layer": {"N": 1, "C": 128, "H": 28, "W": 28, "K": 128, "R": 3, "S": 3, "stride": 1, "padding": 1,
              "dilation": 1},
    "matchings": ["MatchResult(hw_abs_dag:wmma_fp16_fp32, compute:%s, shape:%s)" % (c, s)
                  for c in ("nnn", "ntn", "tnn", "ttn") for s in ("16x16x16", "32x8x16", "8x32x16")],
    "selected": "MatchResult(hw_abs_dag:wmma_fp16_fp32, compute:nnn, shape:8x32x16)",
    "axis_map": {"i": ["n", "n", "n", "p", "p", "q", "q"], "j": ["k"] * 7,
                 "rk": ["rc", "rr", "rs", "rc", "rs", "rc", "rr"]},
    "num_mappings": 35,
    "infeasible": [[0, 0, 0, 0, 0, 0, 1], [0, 0, 0, 0, 1, 0, 0], [0, 0, 0, 0, 1, 0, 1], [0, 0, 1, 0, 0, 0, 0],
                   [0, 0, 1, 0, 0, 0, 1], [0, 0, 1, 0, 1, 0, 0], [0, 0, 1, 0, 1, 0, 1], [0, 1, 0, 0, 0, 0, 0],
                   [0, 1, 0, 0, 0, 0, 1], [0, 1, 0, 0, 1, 0, 0], [0, 1, 1, 0, 0, 0, 0], [1, 0, 0, 0, 0, 0, 0],
                   [1, 0, 1, 0, 0, 0, 0], [1, 1, 0, 0, 0, 0, 0], [1, 1, 1, 0, 0, 0, 0]],
    "num_feasible": 20,
    "first_explored_mapping": [0, 0, 0, 0, 0, 1, 0],
    "trials": {"total": 1200, "rounds": 10, "per_matching": 120, "per_mapping": 6},
}
with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "readme_conv2d_mappings.json"), "w") as f:
    json.dump(fixture, f, indent=1)
