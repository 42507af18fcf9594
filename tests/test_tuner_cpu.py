"""Host logic of the tuning stack on CPU: template sampling, CGA loop, records, failure handling.

The GPU is replaced by a synthetic measurer with the builder/runner interface (set_task,
get_build_kwargs, build, run): latency comes from a closed-form model of the template parameters,
so the search has something to optimise and the tests stay deterministic enough.
"""
import copy
import json
import math
import os
import random
import time

import numpy as np
import pytest

from heron_amd import backend as B
from heron_amd.config import Config
from heron_amd.environment import Env
from heron_amd.multi import Job
from heron_amd.ops.rocm import getOpFromName
from heron_amd.runner import MeasureErrorNo, MeasureResult, Runner, measure_option
from heron_amd.runner.measure import BuildResult
from heron_amd.task import Task


class FakeBuilder:
    n_parallel = 2

    def set_task(self, task, build_kwargs=None):
        self.task = task

    def build(self, inputs):
        out = []
        for inp in inputs:
            s, args = inp.task.instantiate(inp.config)
            err = None if B.check_desc(s.to_desc()) else (MeasureErrorNo.INSTANTIATION_ERROR, "bad desc")
            out.append(BuildResult(s.to_desc().as_tuple(), dict(s.params), None, err, 0.0))
        return out


class FakeRunner:
    """Latency model: bigger tiles and 2 waves/SIMD are faster; one instance family 'fails to launch'."""

    def __init__(self):
        self.calls = 0

    def set_task(self, task):
        return None

    def get_build_kwargs(self):
        return {'check_gpu': {'lds_bytes_per_wg': 163840, 'max_threads_per_wg': 1024, 'wave_size': 64,
                              'regs_per_simd_lane': 512, 'simd_per_cu': 4, 'cu_count': 256}}

    def run(self, inputs, builds):
        res = []
        for inp, br in zip(inputs, builds):
            self.calls += 1
            if br.error is not None:
                res.append(MeasureResult((RuntimeError(br.error[1]),), br.error[0], 0.0, time.time()))
                continue
            p = br.problem
            if p['bm'] == 16 and p['bn'] == 16:
                res.append(MeasureResult((RuntimeError("launch failed"),), MeasureErrorNo.RUNTIME_DEVICE, 0.0, time.time()))
                continue
            cost = 1e-3 * (1 + 64.0 / p['bm'] + 64.0 / p['bn'] + 0.1 * abs(p['stages'] - 3) + (0.3 if p['mfma'] == 16 else 0))
            res.append(MeasureResult(cost, 0, 0.01, time.time()))
        return res


def make_env(tmp_path, method="CGA", trials=48, case=("gemm", [1024, 1024, 1024]), dtype="float16"):
    cfg = Config()
    cfg.codegen_type, cfg.target_name, cfg.get_op = 'GPU_MFMA', 'rocm', getOpFromName
    cfg.out_name = str(tmp_path / "OPS")
    cfg.feasible_file_path = str(tmp_path / "feasible.json")
    cfg.feasible_samples = 48
    cfg.opt_method, cfg.max_trials = method, trials
    cfg.measure_time_per_round, cfg.pop_num, cfg.select_num, cfg.iter_walks = 16, 16, 8, 1
    cfg.parallel_num, cfg.history_topk = 2, 8
    cfg.in_dtype, cfg.out_dtype = dtype, dtype
    env = Env(measure_option(FakeBuilder(), FakeRunner()), cfg)
    op, shape = case
    env.createTask("T1", cfg.get_op(op), shape + [cfg.in_dtype, cfg.out_dtype], cfg.target_name)
    return env


@pytest.mark.parametrize("op,shape,dtype", [("gemm", [8192, 8192, 8192], "float16"), ("gemm", [64, 64, 64], "int8"),
                                            ("bmm", [192, 512, 64, 512], "float16"),
                                            ("c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1], "float16"),
                                            ("c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1, "OhwI64o4i"], "int8"),
                                            ("bmm", [12, 512, 64, 512], "int8")])
def test_every_sampled_instance_passes_the_c_side_check(op, shape, dtype):
    """The Python constraint set and hrn_check_desc describe the same template space."""
    cfg = Config()
    cfg.codegen_type = 'GPU_MFMA'
    t = Task("t", getOpFromName(op), shape + [dtype, dtype], "rocm")
    t.config = cfg
    t.make_stage_schedules()
    assert len(t.knob_manager.knob_names) == 18 and t.knob_manager.sched_tups[0] == ('start', t.knob_manager.sched_tups[0][1])
    seen = set()
    for _ in range(40):
        km = copy.deepcopy(t.knob_manager)
        valid, point = km.randSample({})
        s, args = t.instantiate(km)
        d = s.to_desc()
        assert valid and B.check_desc(d), (d, B.lib().hrn_last_error())
        g = s.info['gemm_view']
        assert d.bm <= 16 * math.ceil(g['M'] / 16) and d.bn <= 16 * math.ceil(g['N'] / 16)
        vals = km.solved_knob_vals_phenotype
        lds_key = [k for k in km.solver.vals if k.endswith("VA:lds_bytes")]
        epi_key = [k for k in km.solver.vals if k.endswith("VA:epi_lds_bytes")][0]
        if d.persistent:                                                       # stages and epilogue region both live
            pkey = [k for k in km.solver.vals if k.endswith("VA:lds_bytes_persistent")][0]
            assert B.lds_bytes(d) == vals[pkey]
        elif d.conv_window:
            # static LDS = the filter stages; the window is dynamic LDS and the epilogue region takes its place later
            assert B.lds_bytes(d) == vals[lds_key[0]]
            win_key = [k for k in km.solver.vals if k.endswith("VA:window_bytes")][0]
            assert vals[win_key] == (d.bm + 2 * (56 + 1)) * (128 if dtype == "float16" else 64)
            assert B.lds_bytes(d) + vals[win_key] <= 163840 - 1024 and B.lds_bytes(d) + vals[epi_key] <= 163840
        else:
            assert B.lds_bytes(d) == max(vals[lds_key[0]], vals[epi_key])
        assert (d.split_k == 1) == (s.params['split_k'] > 1)
        assert [a.name for a in args][-1] == s.info['stage_name']
        seen.add(d.as_tuple())
    assert len(seen) > 20
    # the hand-picked 256x256 instance is inside the space (fp16/int8 GEMM)
    if op == "gemm" and shape[0] == 8192:
        km = copy.deepcopy(t.knob_manager)
        P = lambda n: "P#ST:dense,AX:None,PA:%s" % n
        _, ok = km.validate({P('mfma'): 32, P('wave_m'): 2, P('wave_n'): 2, P('tile_m'): 4, P('tile_n'): 4,
                             P('block_k_bytes'): 128, P('lds_stages'): 2, P('lds_swizzle'): 2})
        assert ok
        _, ok = km.validate({P('mfma'): 32, P('wave_m'): 2, P('wave_n'): 2, P('tile_m'): 4, P('tile_n'): 4,
                             P('block_k_bytes'): 128, P('lds_stages'): 3})
        assert not ok                                            # 192 KiB of LDS


def test_cga_tuning_loop_writes_reference_format(tmp_path):
    env = make_env(tmp_path)
    np.random.seed(0)
    env.tune("T1")
    log = env.config.log_dir
    for f in ("schedule.py", "constraints.py", "records.txt", "stat.txt"):
        assert os.path.exists(os.path.join(log, f)), f
    every = [json.loads(l) for l in open(os.path.join(log, "records.txt"))]
    # the search's own rows carry exactly the reference's keys; the confirmation phase appends rows with one more
    rows = [r for r in every if not r.get("confirmed")]
    assert 30 <= len(rows) <= 48 and len(every) > len(rows)
    for r in every:
        assert set(r) - {"confirmed"} == {"code", "perf", "latency", "time", "param"}
        assert r["perf"] == 0.0 or abs(r["latency"] - math.exp(-r["perf"])) < 1e-12
        assert len(r["code"].split("_")) - 1 == len(r["param"])
    stat = [l.strip().split(",") for l in open(os.path.join(log, "stat.txt"))]
    assert len(stat) == math.ceil(48 / 16) + 1 and all(len(x) == 6 for x in stat)
    # the search found a good point of the synthetic model (optimum 1.5 ms at 256x256, 3 stages)
    best = max(r["perf"] for r in rows)
    assert math.exp(-best) < 2.2e-3
    # failed launches were recorded with perf 0 and kept out of the training data
    assert all(y != 0 for y in env.perf_buffer.data_y)
    # apply_best re-instantiates the best record
    t2 = make_env(tmp_path / "again").task
    s, args = t2.apply_best(os.path.join(log, "records.txt"))
    best_row = max([r for r in every if r.get("confirmed")], key=lambda r: r["perf"])
    assert s.params['bm'] == best_row["param"]["V#ST:dense,AX:None,VA:block_m"]
    assert "mfma" in t2.getStmt(t2.knob_manager)
    # constraints.py is re-loadable and equals the live constraint system
    from heron_amd.schedule.constraints import Solver
    again = Solver.from_dump(open(os.path.join(log, "constraints.py")).read())
    assert len(again.vals) == len(env.task.knob_manager.solver.vals)
    from heron_amd.schedule.constraints.primitives import removedot
    assert again.SATScore({removedot(k): v for k, v in best_row["param"].items()}) == 0


def test_crand_tuner_and_last_round_quirk(tmp_path):
    """max_trials a multiple of the round size: the final round measures nothing (tuner.py:50-58 of the reference)."""
    env = make_env(tmp_path, method="CRAND", trials=32)
    env.tune("T1")
    rows = [json.loads(l) for l in open(os.path.join(env.config.log_dir, "records.txt"))]
    assert len(rows) <= 32
    stat = open(os.path.join(env.config.log_dir, "stat.txt")).read().strip().splitlines()
    assert len(stat) == 3


def test_results2tup_and_error_mapping():
    r = Runner(None)
    res = r.results2tup([MeasureResult(2e-6, 0, 0, 0), MeasureResult((RuntimeError("x"),), MeasureErrorNo.RUN_TIMEOUT, 0, 0),
                         MeasureResult([1e-3, 3e-3], 0, 0, 0), MeasureResult(1e-3, MeasureErrorNo.VERIFY_FAILED, 0, 0)])
    assert res[0] == (0, math.log(1 / 2e-6)) and res[1] == (MeasureErrorNo.RUN_TIMEOUT, 0.0)
    assert abs(res[2][1] - math.log(1 / 2e-3)) < 1e-12 and res[3] == (100, 0.0)


def _sleepy(seconds):
    time.sleep(seconds)
    return [1]


def test_job_timeout_kills_the_child():
    job = Job(_sleepy, (30,), timeout=0.5)
    t0 = time.time()
    job.start(job.attach_info)
    assert job.get() == 0 and time.time() - t0 < 10
    job = Job(_sleepy, (0,), timeout=10)
    job.start(job.attach_info)
    assert job.get() == [1]


def test_cost_model_learns_and_ranks():
    from heron_amd.model import XGBoostCostModel

    class T:
        target = "rocm"

    class S:
        def __init__(self, p):
            self.point = p
    cfg = Config()
    m = XGBoostCostModel(T(), cfg)
    rng = np.random.default_rng(0)
    X = rng.integers(0, 8, (200, 6))
    y = 10 + X[:, 0] * 0.5 - X[:, 3] * 0.3
    assert np.all(m.predict([S(list(x)) for x in X[:5]]) == 1)           # untrained -> ones
    m.fit(X, y)
    pred = m.predict([S(list(x)) for x in X])
    assert np.corrcoef(pred, y)[0, 1] > 0.95
    score = m.bst.get_score()
    assert max(score, key=score.get) in ("f0", "f3")


@pytest.mark.parametrize("op,shape", [("gemv", [4096, 4096]), ("scan", [512, 512, 512]), ("mean", [32, 64, 56, 56]),
                                      ("var", [32, 64, 56, 56]), ("c1d", [32, 1024, 64, 128, 3, 1, 1, 1]),
                                      ("c1d_nwc", [32, 1024, 64, 128, 3, 2, 1, 2]),
                                      ("c2d_nchw", [32, 224, 224, 3, 64, 7, 7, 2, 3, 1]),
                                      ("dil", [16, 56, 56, 64, 64, 3, 3, 1, 2, 2]),
                                      ("c3d", [16, 8, 28, 28, 16, 32, 3, 3, 3, 1, 1, 1]),
                                      ("c3d_ndhwc", [16, 8, 28, 28, 16, 32, 3, 3, 3, (2, 1, 1), 1, 1]),
                                      ("t2d", [16, 14, 14, 64, 32, 4, 4, 2, 1, 1, 0]),
                                      ("dep", [16, 112, 112, 32, 32, 3, 3, 1, 1, 1])])
def test_registry_operators_have_a_feasible_template_space(op, shape):
    """Every operator of the registry (ops/cuda/__init__.py:15-32 names) yields a tunable space on the MFMA templates
    whose samples the C side accepts, and announces kernel operands of the GEMM / conv view it declares."""
    cfg = Config()
    cfg.codegen_type = 'GPU_MFMA'
    t = Task("t", getOpFromName(op), shape + ["float16", "float16"], "rocm")
    t.config = cfg
    t.make_stage_schedules()
    seen = set()
    for _ in range(6):
        km = copy.deepcopy(t.knob_manager)
        valid, _ = km.randSample({})
        s, args = t.instantiate(km)
        d = s.to_desc()
        assert valid and B.check_desc(d), (d, B.lib().hrn_last_error())
        seen.add(d.as_tuple())
        g = s.info['gemm_view']
        p = s.to_problem()
        assert (p.m, p.n, p.k) == (g['M'], g['N'], g['K'])
        assert s.info['adapter'] in __import__('heron_amd.hostops', fromlist=['ADAPTERS']).ADAPTERS
    assert len(seen) >= 3


@pytest.mark.parametrize("method", ["GA", "SRGA", "SDGA", "IDEA", "SA", "CSA", "RCGA"])
def test_baseline_tuners_run_and_only_measure_feasible_points(tmp_path, method):
    """The comparison tuners of the reference's ablations (environment.py:68-91): each completes a run on the CDNA4
    space, every measured record is a feasible point of the CSP, and the search beats the worst tile of the model."""
    env = make_env(tmp_path, method=method, trials=24)
    random.seed(1)
    np.random.seed(1)
    env.tune("T1")
    rows = [json.loads(l) for l in open(os.path.join(env.config.log_dir, "records.txt"))]
    assert 8 <= len(rows) <= 40           # one full round of 16 plus the 24 % 16 remainder round
    solver = env.task.knob_manager.solver
    for r in rows:
        assert solver.SATScore(r["param"]) == 0
    assert math.exp(-max(r["perf"] for r in rows)) < 3.0e-3
    if method in ("GA", "SRGA", "SDGA", "IDEA", "SA"):
        assert os.path.exists(env.config.feasible_file_path)     # per-variable feasible values were sampled first


class _S:
    def __init__(self, predict, violation=0, valid=True, violations=None):
        self.predict, self.violation, self.valid, self.violations = predict, violation, valid, violations


def test_stochastic_ranking_prefers_feasible_then_score():
    from heron_amd.tuner import SRGATuner
    t = SRGATuner.__new__(SRGATuner)
    random.seed(0)
    # all feasible: plain sort by predicted score, best first
    pop = [_S(p) for p in (1.0, 5.0, 3.0, 4.0, 2.0)]
    assert [s.predict for s in t.RankPop(pop)] == [5.0, 4.0, 3.0, 2.0, 1.0]
    # pf = 0: infeasible neighbours are ordered by violation only, so the heavy violator sinks below the light one
    t.PF = 0.0
    pop = [_S(9.0, violation=50), _S(1.0, violation=2), _S(2.0, violation=0)]
    ranked = t.RankPop(pop)
    assert [s.violation for s in ranked] == [0, 2, 50]


def test_idea_rank_fronts_and_sa_acceptance():
    from heron_amd.tuner import IDEATuner, RandomWalkSATuner

    class KM:
        class solver:
            primitives = [0, 1]
    t = IDEATuner.__new__(IDEATuner)
    # (predict, violations): a dominates c (better score, smaller violations); b trades score for violation
    a, b, c = _S(5.0, valid=False, violations=[1, 1]), _S(6.0, valid=False, violations=[3, 3]), _S(4.0, valid=False, violations=[2, 2])
    for s in (a, b, c):
        s.knob_manager = KM
    ranked = t.Rank([c, b, a])
    # objectives are (predict, rank-sum) with larger dominating (idea_tuner.py:96-98): b has the top score and the
    # top rank-sum so it alone forms the first front
    assert ranked[0] is b and {id(x) for x in ranked} == {id(a), id(b), id(c)}
    sa = RandomWalkSATuner.__new__(RandomWalkSATuner)
    np.random.seed(0)
    cur = [_S(1.0) for _ in range(200)]
    better = [_S(2.0) for _ in range(200)]
    worse = [_S(0.5) for _ in range(200)]
    bad = [_S(9.0, valid=False) for _ in range(200)]
    assert all(x.predict == 2.0 for x in sa.accept(cur, better, 0.5))             # improvements always accepted
    frac = np.mean([x.predict == 0.5 for x in sa.accept(cur, worse, 0.5)])
    assert 0.2 < frac < 0.55                                                         # exp(-0.5/0.5) = 0.37
    assert np.mean([x.predict == 0.5 for x in sa.accept(cur, worse, 0.0)]) == 0      # frozen: never
    assert all(x.predict == 1.0 for x in sa.accept(cur, bad, 0.5))                   # infeasible steps rejected


def test_x86_case_forms_with_weight_layout_names_are_accepted():
    """Cases of the DL Boost experiments carry the blocked weight layout's name as a last shape entry
    (tests/figure8/configs/c1d.json, c3d.json, dil.json, t2d.json of the reference)."""
    class Ctx:
        def set_info(self, info):
            self.info = info

        def set_axis_map(self, m):
            pass
    for name, shape in [("c1d", [1, 892, 512, 1024, 1, 1, 0, 1, 'OwI64o4i']), ("c3d", [1, 8, 56, 56, 64, 64, 3, 3, 3, 1, 1, 1, 'OdhwI64o4i']),
                        ("dil", [1, 56, 56, 64, 64, 3, 3, 1, 1, 2, 'OhwI64o4i']), ("t2d", [1, 56, 56, 64, 64, 3, 3, 1, 1, 1, 0, 'OIhw4i16o4i']),
                        ("c2d", [1, 14, 14, 256, 512, 1, 1, 2, 0, 1, 'OhwI48o4i'])]:
        c = Ctx()
        out = getOpFromName(name)(c, *shape, "int8", "int32")
        assert c.info['kind'] == 'u8s8' and out[0].dtype == "int32" and c.info['gemm_view']['K'] % 16 == 0


def test_samples_of_every_registry_operator_survive_the_sampler_processes():
    """Samples are produced in forked children and come back pickled: operator wrappers must not break that."""
    import pickle
    from heron_amd.tuner.tuner import constrained_random_sample_parallel
    cfg = Config()
    cfg.codegen_type, cfg.parallel_num = 'GPU_MFMA', 2
    for op, shape in [("c1d", [16, 892, 512, 512, 3, 1, 4, 1]), ("t2d", [16, 14, 14, 64, 32, 4, 4, 2, 1, 1, 0]), ("gemv", [1024, 256])]:
        t = Task("t", getOpFromName(op), shape + ["float16", "float16"], "rocm")
        t.config = cfg
        t.make_stage_schedules()
        pickle.dumps(t)
        samples = constrained_random_sample_parallel(t, 4, cfg, 60)
        assert len(samples) == 4 and all(s.valid for s in samples)


def test_pretrained_cross_task_model_steers_a_new_task(tmp_path):
    """Records of one GEMM shape train a model that is used, without re-training, to tune another shape of the same
    operator (Tuner.run_with_pretrained, tuner/tuner.py:32-45 of the reference)."""
    env_a = make_env(tmp_path / "a", method="CGA", trials=48)
    env_a.tune("T1")
    rec_a = os.path.join(env_a.config.log_dir, "records.txt")
    env_b = make_env(tmp_path / "b", method="CGA", trials=24, case=("gemm", [2048, 512, 1024]))
    env_b.config.pretrained_records = [rec_a]
    env_b.config.search_generations = 2
    env_b.tune("T1")
    rows = [json.loads(l) for l in open(os.path.join(env_b.config.log_dir, "records.txt"))]
    assert 12 <= len(rows) <= 24
    # the synthetic latency model favours large tiles (1.5e-3 at 256x256, 2.0e-3 at 128x128, above 3e-3 at 64x64 and
    # below); the search is randomly seeded, so the bound leaves room for a 128x128 instance with an off-centre stage count
    assert math.exp(-max(r["perf"] for r in rows)) < 2.3e-3
    stat = open(os.path.join(env_b.config.log_dir, "stat.txt")).read().strip().splitlines()
    assert len(stat) == 2
    # records of another operator family are refused
    from heron_amd.model import PretrainedCostModel
    other = tmp_path / "other_family.txt"
    with open(other, "w") as f:
        for r in rows[:4]:
            f.write(json.dumps(dict(r, param={k.replace("ST:dense", "ST:conv2d_nhwc"): v for k, v in r["param"].items()})) + "\n")
    with pytest.raises(ValueError):
        PretrainedCostModel(env_b.task, env_b.config).fit_from_records([str(other)], 7)


TUNED = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quick_start", "rocm", "tuned")


@pytest.mark.parametrize("rel,op,shape,dtype", [
    ("GEMM_F16_4096/G4096", "gemm", [4096, 4096, 4096], "float16"),
    ("GEMM_F16_8192/G8192", "gemm", [8192, 8192, 8192], "float16"),
    ("GEMM_INT8/G8192", "gemm", [8192, 8192, 8192], "int8"),
    ("BMM_F16/QK", "bmm", [192, 512, 64, 512], "float16"),
    ("BMM_F16/PV", "bmm", [192, 512, 512, 64], "float16"),
    ("C2D_F16/C1", "c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1], "float16"),
    ("C2D_INT8/C1", "c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1, "OhwI64o4i"], "int8")])
def test_shipped_tuned_records_reinstantiate(rel, op, shape, dtype):
    """The records kept for ``run.py -t`` (the 32 best of a search on MI355X per benchmark case and the rows its
    confirmation phase re-timed) are feasible points of
    today's constraint system and Task.apply_best turns the best of them into a template instance the library accepts."""
    path = os.path.join(TUNED, rel, "records.txt")
    rows = [json.loads(l) for l in open(path)]
    plain = [r for r in rows if not r.get("confirmed")]
    assert 1 <= len(plain) <= 32 and all(r["perf"] > 0 for r in rows)
    cfg = Config()
    cfg.codegen_type = 'GPU_MFMA'
    t = Task("t", getOpFromName(op), shape + [dtype, dtype], "rocm")
    t.config = cfg
    t.make_stage_schedules()
    for r in rows:
        assert t.knob_manager.solver.SATScore(dict(r["param"])) == 0
    s, args = t.apply_best(path)
    assert B.check_desc(s.to_desc()), B.lib().hrn_last_error()
    confirmed = [r for r in rows if r.get("confirmed")]
    best = max(confirmed or rows, key=lambda r: r["perf"])          # rows re-timed with long repeats take precedence
    stage = s.info['stage_name']
    assert s.params['bm'] == best["param"]["V#ST:%s,AX:None,VA:block_m" % stage]


def test_refinement_rounds_measure_one_knob_neighbours(tmp_path, capsys):
    """CGA spends the last quarter of its measuring rounds on the one-knob neighbourhood of the best measured points:
    every neighbour is a feasible point that differs from one of the incumbents in exactly one knob, or is the incumbent
    with its wave grid transposed, or one of the operator's coupled moves."""
    env = make_env(tmp_path, method="CGA", trials=48)
    np.random.seed(2)
    random.seed(2)
    env.tune("T1")
    out = capsys.readouterr().out
    assert out.count("refinement round:") == 1                       # 3 measuring rounds of 16 -> the last one
    tuner = env.tuner if hasattr(env, "tuner") else None
    from heron_amd.tuner.ga_tuner import CGATuner
    t = tuner or CGATuner(env.config)
    t.buildCostModel(env.task)
    near = t.incumbent_neighbours(env, top=2)
    assert len(near) >= 10
    solver = env.task.knob_manager.solver
    names = env.task.knob_manager.knob_names
    tops = [s.knob_manager.solved_knob_vals_genotype for s in t.history_topk_samples(env, 2)]
    for s in near:
        vals = s.knob_manager.solved_knob_vals_phenotype
        assert s.valid and solver.SATScore(vals) == 0
        diffs = [[n for n in names if vals[n] != top[n]] for top in tops]
        # one knob away from an incumbent (it may coincide with the other one), its transposed wave grid, or one of the
        # operator's coupled moves (other MFMA edge at the same block tile; other row length, stage count and swizzle)
        coupled = (("wave_m", "wave_n", "tile_m", "tile_n"), ("mfma", "tile_m", "tile_n", "lds_swizzle"),
                   ("block_k_bytes", "lds_stages", "lds_swizzle"), ("issue_order", "load_spread"))
        assert any(len(d) == 1 or (d and any(all(n.endswith(c) for n in d) for c in coupled)) for d in diffs)
    # the share is a config key read at run time; 0 gives the plain loop, and so does any tuner but the constrained GA
    env.config.refine_share = 0
    assert t.refinement_share() == 0.0
    from heron_amd.tuner.random_tuner import CRandTuner
    assert CRandTuner(env.config).refinement_share() == 0.0


def test_stem_reference_inputs_match_the_operator_not_the_padded_kernel():
    """--check on a 3-channel stem: the host reference yields unpadded (N,H,W,3) / (CO,KH,KW,3) arrays while the kernel
    runs on 8 padded channels.  The measurer must take them through the operand adapter (operator layouts), and must
    refuse operands whose shapes differ from what the operator declares."""
    import importlib.util
    from heron_amd.runner import measure_methods as MM
    spec = importlib.util.spec_from_file_location(
        "rocm_run", os.path.join(os.path.dirname(__file__), "quick_start", "rocm", "run.py"))
    run_py = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(run_py)

    class Ctx:
        def set_info(self, info):
            self.info = info

        def set_axis_map(self, m):
            pass

    params = [2, 20, 20, 3, 16, 7, 7, 2, 3, 1, "float16", "float16"]
    ctx = Ctx()
    outs = getOpFromName("c2d")(ctx, *params)
    info = ctx.info
    assert info['adapter'] == 'c2d_krsc' and info['conv']['CI'] == 8
    kernel_shapes = [tuple(t.shape) for t in outs[0].op.input_tensors]
    assert kernel_shapes == [(2, 20, 20, 8), (16, 7, 7, 8)]
    ref_input, ref_output = run_py.host_reference("c2d")(params)
    declared = [tuple(v) for k, v in info['reference_args'].items() if k != 'out']
    assert [tuple(x.shape) for x in ref_input] == declared == [(2, 20, 20, 3), (16, 7, 7, 3)]
    assert tuple(ref_output.shape) == tuple(outs[0].shape)

    class NoCuda:                       # stands in for torch: reaching the upload would be the bug
        float16 = uint8 = int8 = None

    with pytest.raises(ValueError, match="declares"):
        MM._operator_inputs(NoCuda, info, [np.zeros(kernel_shapes[0], np.float16), ref_input[1]])
    with pytest.raises(ValueError, match="operator takes"):
        MM._operator_inputs(NoCuda, info, [ref_input[0]])


def test_analytic_estimate_rewards_co_resident_workgroups():
    """Two points that differ only in how many workgroups fit a CU side by side (LDS of one workgroup): the waiting
    parts of the estimate are paid once per round of co-resident workgroups, so the roomier point must be faster."""
    from heron_amd.schedule.sched_op.mfma_features import analytic_seconds
    info = {'kind': 'f16', 'gemm_view': dict(batch=192, M=512, N=512, K=64)}
    v = dict(mfma=16, wave_m=2, wave_n=2, tile_m=4, tile_n=4, block_k_bytes=128, conv_window=0, persistent=0,
             lds_stages=2, lds_swizzle=2, waves_per_eu=0, epilogue=1, split_k=1, raster_group_m=4, issue_order=1,
             load_spread=2, block_m=128, block_n=128, waves=4, k_steps=2, k_tiles=1, grid_m=4, grid_n=4,
             lds_bytes=65536, window_bytes=0, regs_per_lane=120, loads_per_tile=8)
    two_per_cu = analytic_seconds(info, v)
    one_per_cu = analytic_seconds(info, dict(v, lds_bytes=120000))
    four_per_cu = analytic_seconds(info, dict(v, lds_bytes=32768))
    assert four_per_cu <= two_per_cu < one_per_cu        # (two per CU already reach the HBM floor of this shape)


def test_confirmation_phase_retimes_the_best_tiles_and_apply_best_prefers_it(tmp_path, capsys):
    """The constrained GA ends with a deterministic phase: the best point of each of the best distinct block tiles, its
    transposed wave grid and the other issue order are timed again with long repeats and filed as confirmed records;
    apply_best then ships the best CONFIRMED row even when a short measurement of another point looked better."""
    env = make_env(tmp_path, method="CGA", trials=32)
    env.config.confirm_tiles, env.config.polish_rounds = 3, 0
    np.random.seed(5)
    random.seed(5)
    env.tune("T1")
    out = capsys.readouterr().out
    assert "Confirmation :" in out and "confirmed best" in out
    path = os.path.join(env.config.log_dir, "records.txt")
    rows = [json.loads(line) for line in open(path)]
    confirmed = [r for r in rows if r.get("confirmed")]
    plain = [r for r in rows if not r.get("confirmed")]
    assert 24 <= len(plain) <= 32 and 3 <= len(confirmed) <= 36
    key = lambda r: (r["param"]["V#ST:dense,AX:None,VA:block_m"], r["param"]["V#ST:dense,AX:None,VA:block_n"],
                     r["param"]["P#ST:dense,AX:None,PA:block_k_bytes"])
    tiles = {key(r) for r in confirmed}
    # three block tiles (a transposed wave grid transposes a non-square tile; a coupled move changes the row length)
    assert len({tuple(sorted(t[:2])) for t in tiles}) <= 3
    # every confirmed row is a feasible point; the best tiles of the search are among them
    best_plain = max(plain, key=lambda r: r["perf"])
    assert key(best_plain) in {key(r) for r in confirmed}
    # a lucky short measurement does not decide what ships
    with open(path, "a") as f:
        lucky = dict(min(plain, key=lambda r: r["perf"]), perf=max(r["perf"] for r in rows) + 1.0)
        f.write(json.dumps(lucky) + "\n")
    s, _ = env.task.apply_best(path)
    best_conf = max(confirmed, key=lambda r: r["perf"])
    assert s.params['bm'] == best_conf["param"]["V#ST:dense,AX:None,VA:block_m"]
    assert abs(math.exp(-best_conf["perf"]) - best_conf["latency"]) < 1e-12
    # without confirmed rows the best row of the file ships, as in the reference
    only_plain = str(tmp_path / "plain.txt")
    open(only_plain, "w").write("\n".join(json.dumps(r) for r in plain) + "\n")
    s2, _ = env.task.apply_best(only_plain)
    assert s2.params['bm'] == best_plain["param"]["V#ST:dense,AX:None,VA:block_m"]
    # other tuners have no such phase
    from heron_amd.tuner.random_tuner import CRandTuner
    assert CRandTuner(env.config).confirmation_tiles() == 0
    # the best rows of an earlier search's records join the candidates of a later search's confirmation
    env2 = make_env(tmp_path / "second", method="CGA", trials=16)
    env2.config.confirm_tiles, env2.config.incumbents = 1, [path]
    np.random.seed(6)
    random.seed(6)
    env2.tune("T1")
    rows2 = [json.loads(line) for line in open(os.path.join(env2.config.log_dir, "records.txt"))]
    codes2 = {r["code"] for r in rows2 if r.get("confirmed")}
    assert best_conf["code"] in codes2
    # ... and (polish_rounds is 1 by default) the one-knob neighbours of the best confirmed point were timed as well:
    # every row of the polish step differs from the point it started from in the knob that was changed and in what
    # the constraint system derives from it, and apply_best ships the best of all confirmed rows
    out2 = capsys.readouterr().out
    assert "Polish :" in out2 and out2.index("Polish :") > out2.index("Confirmation :")
    n_conf = int(out2.split("Confirmation : ")[1].split(" ")[0])
    n_polish = int(out2.split("Polish : ")[1].split(" ")[0])
    confirmed2 = [r for r in rows2 if r.get("confirmed")]
    assert n_polish >= 5 and len(confirmed2) == n_conf + n_polish
    s3, _ = env2.task.apply_best(os.path.join(env2.config.log_dir, "records.txt"))
    assert s3.params['bm'] == max(confirmed2, key=lambda r: r["perf"])["param"]["V#ST:dense,AX:None,VA:block_m"]


def test_problem_travels_to_the_measurement_server_without_its_device_pointers():
    """The builder hands the problem to the measuring process as plain integers; the pointers in it (split-K workspace,
    caller-supplied column sums) belong to the process that launches and stay behind."""
    from heron_amd import backend as B
    from heron_amd.runner import measure_methods as MM
    d = MM._problem_to_dict(B.gemm_problem(2, 100, 200, 64, 8, split_k=2))
    assert d['m'] == 100 and d['n'] == 200 and d['k'] == 64 and d['batch'] == 2 and d['split_k'] == 2
    assert all(isinstance(v, int) for v in d.values())
    assert not {'workspace', 'workspace_bytes', 'bsum'} & set(d)


def test_variable_ranking_follows_the_boosters_feature_weights():
    from heron_amd.utils import anaCostModel

    class Booster:
        def get_score(self, importance_type='weight'):
            return {'f2': 5.0, 'f0': 1.0, 'f3': 5.0}

    class Model:
        bst = Booster()

    assert anaCostModel(Model, list('abcde')) == ['c', 'd', 'a', 'b', 'e']
    Model.bst = None
    assert sorted(anaCostModel(Model, list('abcde'))) == list('abcde')


def test_coupled_moves_reach_the_other_row_length_and_the_other_mfma_edge():
    """From a 256x256 tile with 64-byte rows, four stages and 16x16 MFMAs, the refinement neighbourhood contains the same
    block tile with 128-byte rows and two stages, and the same block tile built from 32x32 MFMAs: feasible points that
    are three knobs away, so no one-knob move finds them."""
    from heron_amd.sample import Sample
    cfg = Config()
    cfg.codegen_type = 'GPU_MFMA'
    t = Task("t", getOpFromName("gemm"), [8192, 8192, 8192, "int8", "int8"], "rocm")
    t.config = cfg
    t.make_stage_schedules()
    km = Sample(t).knob_manager
    names = km.knob_names
    want = dict(mfma=16, wave_m=4, wave_n=2, tile_m=4, tile_n=8, block_k_bytes=64, lds_stages=4, lds_swizzle=3, persistent=0,
                split_k=1, conv_window=0, epilogue=1, column_sums=1)
    knobs = {}
    for n in names:
        short = n.split("PA:")[-1]
        knobs[n] = want.get(short, km.get_knob_candidates(n)[0])
    point, valid = km.validate(knobs)
    assert valid
    labelled = t.coupled_moves(km)
    assert {label for label, _ in labelled if not label.startswith("issue_order")} == {"mfma=32", "block_k_bytes=128", "block_k_bytes=256"}
    assert len({label for label, _ in labelled if label.startswith("issue_order=")}) == 4        # the other order x 4 spreads
    moves = [m for _, m in labelled]

    def short(d):
        return {n.split("PA:")[-1]: v for n, v in d.items()}

    feasible = []
    for m in moves:
        p, ok = Sample(t).knob_manager.validate(m)
        if ok:
            feasible.append(short(m))
    assert any(m['block_k_bytes'] == 128 and m['lds_stages'] == 2 and m['mfma'] == 16 and m['tile_m'] == 4 for m in feasible)
    assert any(m['mfma'] == 32 and m['tile_m'] == 2 and m['tile_n'] == 4 and m['block_k_bytes'] == 64 for m in feasible)
    # every move keeps the block tile: rows per wave tile x wave grid unchanged
    assert all(m['tile_m'] * m['mfma'] == 64 and m['tile_n'] * m['mfma'] == 128 for m in map(short, moves))
