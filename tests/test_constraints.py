"""Constraint primitives, the finite-domain solver and the KnobManager.

Known-answer fixtures: the reference's committed dumps of the 64^3 GEMM search spaces (59 variables for
its DL Boost template, 172 for its TensorCore template) with the 32 measured - hence feasible -
parameter sets of each run (tests/golden/*_gemm64_csp.json, written by make_constraint_fixtures.py).
"""
import json
import os
import random

import pytest

from heron_amd.schedule.constraints import EQ, LE, LT, NE, KnobManager, ProdTwo, Solver, Sum

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(plat):
    spec = json.load(open(os.path.join(GOLD, "%s_gemm64_csp.json" % plat)))
    return Solver.from_spec(spec), spec["records"]


def as_point(param):
    return {k.replace('.', '_'): v for k, v in param.items()}


@pytest.mark.parametrize("plat,nvars,ncons", [("dlboost", 59, 55), ("tensorcore", 172, 199)])
def test_reference_records_satisfy_our_evaluators(plat, nvars, ncons):
    s, records = load(plat)
    assert len(s.vals) == nvars and len(s.primitives) == ncons and len(records) == 32
    for r in records:
        p = as_point(r["param"])
        assert set(p) == set(s.vals)
        assert s.in_bounds(p)
        scores, valid = s.MultiSATScore(p)
        assert valid and s.SATScore(p) == 0
        # records.txt semantics: perf = ln(1/seconds)
        assert abs(r["latency"] - __import__("math").exp(-r["perf"])) < 1e-12


@pytest.mark.parametrize("plat", ["dlboost", "tensorcore"])
def test_broken_records_are_caught(plat):
    """Perturbing one split factor of a feasible point must violate a product constraint."""
    s, records = load(plat)
    random.seed(1)
    caught = 0
    for r in records[:8]:
        p = as_point(r["param"])
        key = random.choice([k for k in p if k.endswith("_inner") or k.endswith("_outer")])
        p[key] = p[key] * 2 + 1
        caught += s.SATScore(p) > 0
    assert caught == 8


@pytest.mark.parametrize("plat,n", [("dlboost", 40), ("tensorcore", 6)])
def test_solver_samples_feasible_points_of_reference_spaces(plat, n):
    s, records = load(plat)
    random.seed(0)
    seen = set()
    for _ in range(n):
        valid, point = s.solve({}, {})
        assert valid
        d = dict(zip(s.vals.keys(), point))
        assert s.in_bounds(d) and s.SATScore(d) == 0
        seen.add(tuple(point))
    assert len(seen) > n // 2            # a sampler, not a constant
    # a full record is accepted, a record with a wrong value is rejected
    p = as_point(records[0]["param"])
    assert s.validate(p)[0]
    bad = dict(p)
    k = [k for k in bad if k.endswith("_inner")][0]
    bad[k] = bad[k] + 1 if bad[k] + 1 <= s.vals[k].up else bad[k] - 1
    assert not s.validate(bad)[0]


def test_known_and_bounds_and_hints_dlboost():
    s, records = load("dlboost")
    p1, p2 = as_point(records[0]["param"]), as_point(records[5]["param"])
    key = "dense_global_j_c_inner"
    for _ in range(5):
        valid, point = s.solve({}, {key: [p1[key], p2[key]]})
        d = dict(zip(s.vals.keys(), point))
        assert valid and d[key] in (p1[key], p2[key])
    valid, point = s.solve({}, {}, {"dense_unroll_pragma": [2, 3]})
    assert valid and 2 <= dict(zip(s.vals.keys(), point))["dense_unroll_pragma"] <= 3
    valid, point = s.solve({"dense_unroll_pragma": 4}, {})
    assert valid and dict(zip(s.vals.keys(), point))["dense_unroll_pragma"] == 4     # hints are honoured when feasible
    valid, point = s.repair(p1)
    assert valid and dict(zip(s.vals.keys(), point)) == p1                            # repairing a feasible point keeps it
    assert s.solve({}, {key: [7]}) == (False, None)                                    # 7 does not divide 64


def test_primitive_scores():
    v = {"a": 6, "b": 3, "c": 2, "z": 0, "o": 1}
    assert ProdTwo(["a", ["b", "c"]]).eval(v) == 0 and ProdTwo(["a", ["b", "b"]]).eval(v) == 3
    assert Sum(["a", ["b", "c", 1]]).eval(v) == 0 and Sum([1, ["z", "o"]]).eval(v) == 0
    assert EQ(["b", 3]).eval(v) == 0 and EQ(["b", "c"]).eval(v) == 1
    assert EQ(["b", "c"], cond="z").eval(v) == 0 and EQ(["b", "c"], cond="o").eval(v) == 1
    assert NE(["b", "c"]).eval(v) == 0 and NE(["b", 3]).eval(v) == 1
    assert LE(["c", "b"]).eval(v) == 0 and LE(["b", "c"]).eval(v) == 1 and LE(["b", 3]).eval(v) == 0
    assert LT(["c", "b"]).eval(v) == 0 and LT(["b", 3]).eval(v) == 1


def test_dump_round_trip():
    s, _ = load("dlboost")
    s2 = Solver.from_dump(s.dump())
    assert list(s2.vals) == list(s.vals) and len(s2.primitives) == len(s.primitives)
    assert s2.dump() == s.dump()
    assert "model.AddMultiplicationEquality(64, [dense_i_outer, dense_i_inner])" in s.dump()


def test_knob_manager_builders_and_operators():
    km = KnobManager()
    km.define_value("P#x", 1, 64, 1, True)
    km.define_value("P#y", 1, 64, 1, True)
    km.addCandidates("P#x", [1, 2, 4, 8, 16, 32, 64])
    km.addCandidates("P#y", [1, 2, 4, 8, 16, 32, 64])
    km.define_value("V#xy", 1, 64, 1)
    km.addProd(["P#x", "P#y"], "V#xy")
    km.addLE("V#xy", 32)
    km.define_value("P#sel", 0, 2, 0, True)
    km.define_value("V#picked", 1, 64, 1)
    km.addSelect(["P#x", "P#y", 5], "P#sel", "V#picked")
    km.addNE("P#x", "P#y")
    km.is_building = False
    random.seed(0)
    pts = []
    for _ in range(20):
        valid, point = km.randSample({})
        v = dict(km.solved_knob_vals_phenotype)
        assert valid and v["P#x"] * v["P#y"] == v["V#xy"] <= 32 and v["P#x"] != v["P#y"]
        assert v["V#picked"] == [v["P#x"], v["P#y"], 5][v["P#sel"]]
        pts.append(tuple(point))
    assert len(set(pts)) > 5
    # constrained crossover: the children take key variables from the parents and stay feasible
    import copy
    m1, m2 = copy.deepcopy(km), copy.deepcopy(km)
    m1.randSample({}); m2.randSample({})
    child = copy.deepcopy(km)
    for _ in range(10):
        point, valid = child.constrained_crossover_and_mutate(m1, m2, ["P#x", "P#sel"])
        v = child.solved_knob_vals_phenotype
        assert valid and child.solver.SATScore(v) == 0
    point, valid = child.constrained_random_walk(m1, 0.3)
    assert valid and child.solver.SATScore(child.solved_knob_vals_phenotype) == 0
    _, ok = child.validate({"P#x": 8, "P#y": 8})
    assert not ok                                               # 64 > 32 and x == y


def test_status_distinguishes_proven_from_given_up():
    """'infeasible' is only claimed when propagation or an exhaustive search proves it; a search that merely sampled
    a wide interval, or ran out of its fail budget, reports 'unknown'."""
    s = Solver()
    s.addVal("x", 0, 3, 0)
    s.addVal("y", 0, 3, 0)
    s.primitives.append(LT(["x", "y"]))
    s.primitives.append(LT(["y", "x"]))
    ok, _ = s.solve({}, {})
    assert not ok and s.last_status == 'infeasible'
    # one feasible value in a wide interval that propagation cannot single out (x*x == y*y + 2001 has the integer
    # solutions x = 1001, y = 1000 only... the solver either finds it or must say that it does not know)
    t = Solver()
    t.addVal("x", 0, 5000, 0)
    t.addVal("y", 0, 5000, 0)
    t.addVal("xx", 0, 25000000, 0)
    t.addVal("yy", 0, 25000000, 0)
    t.primitives.append(ProdTwo(["xx", ["x", "x"]]))
    t.primitives.append(ProdTwo(["yy", ["y", "y"]]))
    t.primitives.append(Sum(["xx", ["yy", 2001]]))
    t.fail_budget, t.restarts = 20, 2
    random.seed(5)
    ok, point = t.solve({}, {})
    if ok:
        assert point[0] == 1001 and point[1] == 1000
    else:
        assert t.last_status == 'unknown'
