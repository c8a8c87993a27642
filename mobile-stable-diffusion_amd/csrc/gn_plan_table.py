#!/usr/bin/env python3
"""Writes gn_plan_table.inc, the table of measured GroupNorm launch plans that gn_plan.hip looks
shapes up in, from the output of one or more sweeps:

    python bench.py --no-cpu --tables gn_plan_sweep --sweep-batches 1,2,4,8,16,32 > sweep.json   (on the GPU)
    python mobile-stable-diffusion_amd/csrc/gn_plan_table.py sweep.json [more.json ...]            (anywhere)

Every sweep row holds, for one shape (element size, vectors per unit, units, output in place or
apart), the time of the plan the library picked (`auto`) and of every plan the knobs could force.
Per distinct shape (rows of the same key are averaged):

  * the candidate is the plan the library picked when the sweep ran, unless that plan is more
    than 3 % behind the fastest measured one - then the fastest.  (The same 3 % the sweep's
    auto_vs_best criterion uses: a shape changes plan only for a gain the criterion can see.)
  * the rule alone (gn_decide with MSD_TUNE_GN_PLAN_RULE_ONLY, asked from the built library: host
    arithmetic) gives its plan for the shape.  No row is written when the rule already picks the
    candidate.  At the batches the library is tuned for (1, 2 and 32: 32, 64 and 1024 units) any
    other difference becomes a row; elsewhere only a rule plan more than 1 % slower than the
    candidate, or one the sweep did not time.

The table is only consulted on the chip it was measured on (256 CUs in 8 XCDs).
"""
import importlib
import json
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(os.path.dirname(HERE))
TUNED_UNITS = (32, 64, 1024)   # batch 1, 2, 32 at 32 groups
KEEP_WITHIN = 1.03             # the shipped plan stays unless it is further than this from the fastest
RULE_MARGIN = 1.01             # away from the tuned batches: a row only if the rule loses more than this


def parse(text):
    m = re.match(r"(\d+)x(\d+)x(\d+)(?: w(\d+))?$", text)
    return int(m.group(1)), int(m.group(2)), int(m.group(3)), int(m.group(4) or 1)


def load_rows(paths):
    rows = []
    for path in paths:
        with open(path) as f:
            for line in f:
                line = line.strip()
                if line.startswith("{"):
                    rows += json.loads(line).get("gn_plan_sweep", [])
                elif line.startswith("["):
                    rows += json.loads(line)
    return rows


def rule_plan(msd, lib, row):
    """The plan of the rule alone for the shape of a sweep row (split, threads, k, writers)."""
    code = msd.DTYPE_F16 if row["dtype"] == "f16" else msd.DTYPE_F32
    assert lib.msd_set_tuning(msd.TUNE_GN_PLAN_RULE_ONLY, 1) == 0
    try:
        return msd.groupnorm_plan(row["batch"], row["c"], row["hw"], 32, code, in_place=row["in_place"])
    finally:
        lib.msd_set_tuning(msd.TUNE_GN_PLAN_RULE_ONLY, 0)


def main(paths, out_path=None):
    sys.path.insert(0, REPO)
    msd = importlib.import_module("mobile-stable-diffusion_amd")
    lib = msd.load_library()
    shapes = {}
    for row in load_rows(paths):
        key = (2 if row["dtype"] == "f16" else 4, 0 if row["in_place"] else 1, row["vectors_per_unit"], row["units"])
        s = shapes.setdefault(key, {"times": {}, "auto": parse(row["auto"]), "rule": rule_plan(msd, lib, row)})
        for text, us in row["variants"].items():
            s["times"].setdefault(parse(text), []).append(us)
    out = []
    for key in sorted(shapes):
        s = shapes[key]
        times = {plan: sum(v) / len(v) for plan, v in s["times"].items()}
        best = min(times, key=times.get)
        shipped = s["auto"]
        cand = shipped if shipped in times and times[shipped] <= KEEP_WITHIN * times[best] else best
        rule = s["rule"]
        if rule == cand:
            continue
        elt, apart, vectors, units = key
        if units not in TUNED_UNITS and rule in times and times[rule] <= RULE_MARGIN * times[cand]:
            continue
        rule_us = "%.2f" % times[rule] if rule in times else "not timed"
        out.append("    {%d, %d, %5d, %4d, %d, %4d, %d},  // %.2f us; the rule: %dx%dx%d%s, %s us" % (
            elt, apart, vectors, units, cand[0], cand[1], cand[3], times[cand], rule[0], rule[1], rule[2],
            " w%d" % rule[3] if rule[3] > 1 else "", rule_us))
    header = ["// Measured GroupNorm launch plans (written by gn_plan_table.py from bench.py --tables gn_plan_sweep;",
              "// do not edit by hand).  {bytes per element, output apart from the input, vectors per unit, units,",
              "// slices per unit, lanes, writers per unit}, then the measured time and what the rule alone picks.",
              "// %d rows from %d measured shapes." % (len(out), len(shapes))]
    with open(out_path or os.path.join(HERE, "gn_plan_table.inc"), "w") as f:
        f.write("\n".join(header + out) + "\n")
    print("%d rows from %d shapes" % (len(out), len(shapes)))
    return out


if __name__ == "__main__":
    if len(sys.argv) < 2:
        sys.exit(__doc__)
    main(sys.argv[1:])
