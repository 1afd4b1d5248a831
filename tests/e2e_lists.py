"""The reference's end-to-end problem lists (tests/golden/e2e_problems.json, written by
tests/golden/make_e2e_lists.py from mlir/test/e2e/*.toml) as option strings."""
import itertools
import json
import os
import re

HERE = os.path.dirname(os.path.abspath(__file__))


def expand(entry):
    """[option string] of one list: its axes multiplied out over its configurations, minus each configuration's
    exclusions, configuration first and axis options behind it (mlir/test/e2e/generateE2ETest.py:123-151).  Like
    that script (:137-139) it leaves out the int8 element type for the two gradients: the reference generates
    int8 for forward convolutions only."""
    out = []
    axes = entry["axes"]
    for test in entry["tests"]:
        excluded = test.get("exclude", {})
        for combo in itertools.product(*[a["values"] for a in axes]):
            if any(v in excluded.get(a["name"], ()) for a, v in zip(axes, combo)):
                continue
            parts = [a["prefix"] + v for a, v in zip(axes, combo)]
            if len(parts) >= 3 and "i8" in parts[2] and ("conv_bwd_data" in parts[0] or "conv_bwd_weight" in parts[0]):
                continue
            out.append(re.sub(r"\s+", " ", " ".join([test["config"]] + parts + [entry["fixed"]])).strip())
    return out


def problems():
    """[(list name, option string)], every problem of every list"""
    with open(os.path.join(HERE, "golden", "e2e_problems.json")) as f:
        lists = json.load(f)
    return [(entry["list"], opts + " -arch gfx950") for entry in lists for opts in expand(entry)]
