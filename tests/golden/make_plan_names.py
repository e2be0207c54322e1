#!/usr/bin/env python3
"""Writes tests/golden/plan_names.json: the kernel routing of every pinned call
(tests/plan_cases.py) as the library reports it through dragon_hip_plan_name. Run it
after a routing change that is meant, and read the diff: a BASELINE shape that moves to
a multi-pass fallback shows up there. Needs no GPU."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from dragon_amd import kernels as K  # noqa: E402
from tests.plan_cases import CASES  # noqa: E402


def main():
    out = {}
    for name, calls in sorted(CASES.items()):
        out[name] = {"%s %s %s %s" % (op, dt, "x".join(str(d) for d in dims), layout):
                     K.plan_name(op, dt, dims, layout) for op, dt, dims, layout in calls}
    path = os.path.join(ROOT, "tests", "golden", "plan_names.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1, sort_keys=True)
        f.write("\n")
    print("wrote", path)


if __name__ == "__main__":
    main()
