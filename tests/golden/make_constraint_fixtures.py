"""Writes tests/golden/{dlboost,tensorcore}_gemm64_csp.json from the reference's committed tuning dumps.

Run in a container that has the reference checkout:  python tests/golden/make_constraint_fixtures.py
It READS the dumps as text (nothing from the reference is imported or executed):
  tests/quick_start/<platform>/OPS/GEMM/G1/constraints.py  - the dumped CSP (variables, bounds, constraints)
  tests/quick_start/<platform>/OPS/GEMM/G1/records.txt     - 32 measured, hence feasible, points
and stores them as data: {"vars": [[name, low, up]], "cons": [[kind, args, cond]], "records": [{"perf", "param"}]}.
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from heron_amd.schedule.constraints.solver import Solver  # noqa: E402

REF = os.environ.get("HERON_REFERENCE", "/root/reference")

for plat in ("dlboost", "tensorcore"):
    base = os.path.join(REF, "tests/quick_start/%s/OPS/GEMM/G1" % plat)
    solver = Solver.from_dump(open(os.path.join(base, "constraints.py")).read())
    spec = solver.to_spec()
    spec["vars"] = [v[:3] for v in spec["vars"]]
    spec["records"] = []
    for line in open(os.path.join(base, "records.txt")):
        row = json.loads(line)
        spec["records"].append({"perf": row["perf"], "latency": row["latency"], "code": row["code"],
                                "param": row["param"]})
    out = os.path.join(HERE, "%s_gemm64_csp.json" % plat)
    with open(out, "w") as f:
        json.dump(spec, f, separators=(",", ":"))
    print(out, len(spec["vars"]), "vars", len(spec["cons"]), "constraints", len(spec["records"]), "records")
