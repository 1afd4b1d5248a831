#!/usr/bin/env python3
"""Writes tests/golden/e2e_problems.json: the problems of the reference's end-to-end test lists
(mlir/test/e2e/*.toml) -- per list its axes (operation, layouts, element types, transposes, perf_config,
store method), its configurations with their exclusions, and the rocmlir-gen options of its suffix;
tests/e2e_lists.py multiplies the axes out into the option strings rocmlir-gen is run with, the way
mlir/test/e2e/generateE2ETest.py does.  Lit substitutions and the
pipeline behind rocmlir-gen are dropped; what is kept of each list's suffix are the rocmlir-gen options in it
(operation, element type, thresholds).  Run in the build container, where /root/reference is mounted:

    python3 tests/golden/make_e2e_lists.py
"""
import glob
import json
import os
import re

import tomli

REF = "/root/reference/mlir/test/e2e"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "e2e_problems.json")
# lists for other architectures' instruction sets
SKIP = {"conv_regression_fwd_navi3x.toml"}


def gen_options(suffix):
    """rocmlir-gen's own options in a list's suffix: everything before the first pipe, lit substitutions removed"""
    head = suffix.split("|")[0]
    toks = [t for t in head.split() if not t.startswith("%")]
    out, i = [], 0
    while i < len(toks):
        t = toks[i]
        if t in ("--arch", "-arch"):      # "--arch %arch": the substitution is already gone
            i += 1
            continue
        out.append(t)
        i += 1
    return " ".join(out)


def main():
    lists = []
    for path in sorted(glob.glob(os.path.join(REF, "*.toml"))):
        name = os.path.basename(path)
        if name in SKIP:
            continue
        doc = tomli.load(open(path, "rb"))
        tests = []
        for suite in doc.get("suite", []):
            for test in suite.get("test", []):
                entry = {"config": re.sub(r"\s+", " ", test["config"]).strip()}
                if test.get("exclude"):
                    entry["exclude"] = {e["name"]: e["values"] for e in test["exclude"]}
                tests.append(entry)
        lists.append({"list": name, "fixed": gen_options(doc.get("suffix", "")),
                      "axes": [{"name": a["name"], "prefix": a.get("prefix", ""), "values": a["values"]}
                               for a in doc.get("axis", [])],
                      "tests": tests})
    with open(OUT, "w") as f:
        json.dump(lists, f, indent=1)
        f.write("\n")
    print(len(lists), "lists ->", OUT)


if __name__ == "__main__":
    main()
