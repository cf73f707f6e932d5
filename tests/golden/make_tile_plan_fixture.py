"""Reduces the timings written by `python bench.py --plan-sweep abc --plan-sweep-out sweep.json`
(run on an MI355X) to the fixture tests/test_tile_plan.py ranks the planner against:
every third problem the tile kernel serves, with the microseconds of each plan timed.

    python tests/golden/make_tile_plan_fixture.py sweep.json [more.json ...]
"""
import json
import os
import sys


def main(paths):
    problems = []
    for p in paths:
        with open(p) as f:
            problems += [r for r in json.load(f) if r.get("plans") and r["own_plan"][0]]
    kept = [dict(kind=r["kind"], M=r["M"], N=r["N"], K=r["K"], plans=r["plans"]) for r in problems[::3]]
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "tile_plan_sweep.json")
    with open(out, "w") as f:
        json.dump(kept, f, separators=(",", ":"))
    print(f"{len(kept)} of {len(problems)} problems -> {out}")


if __name__ == "__main__":
    main(sys.argv[1:])
