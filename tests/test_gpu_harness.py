"""The harnesses around the kernels, on the GPU and with every measured kernel verified against a host reference:
the network driver (tests/network/run.py; per-layer tuning, plain and count-weighted sums, the reference's
``Case ..., Times : n, latency ...`` lines of tests/figure10/run.py:105-109), every baseline search method with the HIP
measurer (tuner/{ga,idea,sa}_tuner.py of the reference), and a search steered by a cost model fitted on the shipped
records of another shape (Tuner.run_with_pretrained, tuner/tuner.py:32-45)."""
import json
import math
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import oracle
from heron_amd import tuned, workloads

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_network_driver_two_layers(hrn, tmp_path):
    cfg = {"config": {"out_name": "OPS/TinyNet", "method": "CGA", "max_trials": 8, "runner_number": 2, "runner_repeat": 3,
                      "runner_timeout": 50, "build_timeout": 50, "in_dtype": "float16", "out_dtype": "float16",
                      "pop_num": 24, "select_num": 12, "iter_walks": 2, "parallel_num": 2, "measure_time_per_round": 8,
                      "cases": {"layer-0": ["c2d", [2, 14, 14, 64, 64, 3, 3, 1, 1, 1], 3],
                                "layer-1": ["gemm", [64, 256, 128], 2]}}}
    path = tmp_path / "tiny.json"
    path.write_text(json.dumps(cfg))
    out = tmp_path / "tiny_out.json"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "network", "run.py"), "-c", str(path), "-m", "8", "--check",
                        "-o", str(out)], cwd=tmp_path, capture_output=True, text=True, timeout=400)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    lines = re.findall(r"^Case (\[.*?\]), Times : (\d+), latency ([0-9.]+) ms\.$", r.stdout, flags=re.M)
    assert [int(t) for _, t, _ in lines] == [3, 2] and all(float(lat) > 0 for _, _, lat in lines)
    plain = float(re.search(r"^Estimated network latency :\s+([0-9.e-]+)$", r.stdout, flags=re.M).group(1))
    weighted = float(re.search(r"^Estimated network latency weighted by layer counts :\s+([0-9.e-]+)$", r.stdout, flags=re.M).group(1))
    lat = [float(x) for _, _, x in lines]
    assert abs(plain - sum(lat)) < 1e-5 and abs(weighted - (3 * lat[0] + 2 * lat[1])) < 1e-5
    assert r.stdout.count("PASS") == 2
    table = json.load(open(out))
    assert [row["times"] for row in table["layers"]] == [3, 2] and abs(table["weighted_sum_ms"] - weighted) < 1e-5
    # every record of both layers was verified against the host reference inside the measurer: none failed
    for layer in ("layer-0", "layer-1"):
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / "TinyNet" / layer / "records.txt")]
        assert rows and all(row["perf"] > 0 for row in rows)


def test_operator_sweep_driver_on_two_case_files(hrn, tmp_path):
    """tests/ops_sweep/run.py (the counterpart of the reference's tests/figure6/run.py and tests/figure8/run.py) on
    two small case files, every measured kernel verified: one table row per case, positive latencies, no record of
    either search marked wrong."""
    common = {"method": "CGA", "max_trials": 8, "runner_number": 2, "runner_repeat": 3, "runner_timeout": 50,
              "build_timeout": 50, "pop_num": 24, "select_num": 12, "iter_walks": 2, "parallel_num": 2,
              "measure_time_per_round": 8, "confirm_tiles": 2}
    cfgs = tmp_path / "cfgs"
    cfgs.mkdir()
    (cfgs / "f16_gemm.json").write_text(json.dumps({"config": dict(common, out_name="OPS/F16_GEMM", in_dtype="float16",
                                                                   out_dtype="float16",
                                                                   cases={"G1": ["gemm", [96, 256, 128]]})}))
    (cfgs / "int8_c2d.json").write_text(json.dumps({"config": dict(common, out_name="OPS/INT8_C2D", in_dtype="int8",
                                                                   out_dtype="int32",
                                                                   cases={"C1": ["c2d", [2, 14, 14, 32, 48, 3, 3, 1, 1, 1, "OhwI32o4i"]],
                                                                          "C2": ["c2d", [1, 9, 9, 16, 16, 1, 1, 1, 0, 1, "OhwI32o4i"]]})}))
    out = tmp_path / "sweep.json"
    r = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "ops_sweep", "run.py"), "--configs", str(cfgs), "-m", "8",
                        "--check", "-o", str(out)], cwd=tmp_path, capture_output=True, text=True, timeout=500)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    table = json.load(open(out))
    assert [(row["config"], row["case"]) for row in table] == [("f16_gemm", "G1"), ("int8_c2d", "C1"), ("int8_c2d", "C2")]
    assert all(row["latency_ms"] > 0 for row in table) and r.stdout.count("PASS") == 3
    for rel in ("F16_GEMM/G1", "INT8_C2D/C1", "INT8_C2D/C2"):
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / rel / "records.txt")]
        assert rows and all(row["perf"] > 0 for row in rows), rel        # error 100 (wrong result) would give perf 0
        assert any(row.get("confirmed") for row in rows), rel


def test_network_replay_as_one_stream_and_as_one_graph(hrn, tmp_path):
    """tests/network/replay.py on the BERT case file: the tuned layers run as one sequence on a stream and from a HIP
    graph; the driver itself compares every checked graph replay with the eager results and fails on a difference."""
    net = os.path.join(ROOT, "tests", "network")
    out = tmp_path / "replay.json"
    r = subprocess.run([sys.executable, os.path.join(net, "replay.py"), "-c", os.path.join(net, "configs", "bert.json"),
                        "-T", os.path.join(net, "tuned", "bert"), "--reps", "5", "--rounds", "3", "-o", str(out)],
                       cwd=tmp_path, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    res = json.load(open(out))
    assert res["layers"] == 3 and res["launches"] == 84 and res["graph_rounds_checked"] == 3
    assert 0 < res["graph_us"] < 3 * res["isolated_sum_us"] and 0 < res["stream_us"] < 3 * res["isolated_sum_us"]


def _env(tmp_path, method, trials, case=("gemm", [64, 64, 64]), dtype=("int8", "int32")):
    from heron_amd.config import Config
    from heron_amd.environment import Env
    from heron_amd.ops.rocm import getOpFromName
    from heron_amd import runner as R
    cfg = Config()
    cfg.codegen_type, cfg.target_name, cfg.get_op = 'GPU_MFMA', 'rocm', getOpFromName
    cfg.out_name = str(tmp_path / "OPS")
    cfg.opt_method, cfg.max_trials, cfg.measure_time_per_round = method, trials, 8
    cfg.pop_num, cfg.select_num, cfg.iter_walks, cfg.parallel_num = 24, 12, 2, 2
    cfg.feasible_samples, cfg.feasible_file_path = 64, str(tmp_path / "feasible.json")
    cfg.in_dtype, cfg.out_dtype = dtype
    runner = R.LocalRunner(number=2, repeat=3, min_repeat_ms=0, timeout=60)
    builder = R.LocalBuilder(timeout=60, n_parallel=4)
    env = Env(R.measure_option(builder, runner), cfg)
    op, shape = case
    task = env.createTask("T1", getOpFromName(op), shape + list(dtype), 'rocm')
    return env, task, runner, builder


@pytest.mark.parametrize("method", ["GA", "SRGA", "SDGA", "IDEA", "SA"])
def test_baseline_tuner_on_the_gpu(method, hrn, tmp_path):
    """Eight verified trials of each baseline search method on the 64^3 quantized GEMM: points the method knows to
    violate the constraints are not built; everything that is measured must run and match the int64 reference."""
    env, task, runner, builder = _env(tmp_path, method, 8)
    try:
        def ref(args):
            A, Bm = workloads.gemm_u8s8_inputs(64, 64, 64, seed=0)
            return [A, Bm], oracle.gemm_int64_numpy(A, Bm)
        task.set_verify_func(ref, rtol=1e-6)
        env.tune("T1")
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / "T1" / "records.txt")]
        assert 1 <= len(rows) <= 16
        assert all(row["perf"] > 0 for row in rows), [row["perf"] for row in rows]
        assert math.exp(-max(row["perf"] for row in rows)) < 100e-6
    finally:
        runner.close()
        builder.close()


def test_pretrained_model_from_shipped_records(hrn, tmp_path):
    """The records shipped for the 4096^3 fp16 GEMM steer the search of a 1024^3 task from its first round, without
    re-training; every measured kernel is verified."""
    env, task, runner, builder = _env(tmp_path, "CGA", 16, case=("gemm", [1024, 1024, 1024]), dtype=("float16", "float16"))
    try:
        env.config.pretrained_records = [tuned.records_path("gemm_f16_4096")]
        env.config.search_generations = 2

        def ref(args):
            A, Bm = workloads.gemm_f16_inputs(1024, 1024, 1024, seed=1)
            return [A, Bm], oracle.gemm_f32(A, Bm)
        task.set_verify_func(ref, rtol=1e-2)
        env.tune("T1")
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / "T1" / "records.txt")]
        assert 8 <= len(rows) <= 16 and all(row["perf"] > 0 for row in rows)
        stat = open(tmp_path / "OPS" / "T1" / "stat.txt").read().strip().splitlines()
        assert len(stat) == 2                                          # two rounds, no re-training between them
        best = math.exp(-max(row["perf"] for row in rows))
        assert 2.0 * 1024 ** 3 / best / 1e12 > 60       # sanity only: 16 trials of a random search (measured 120-260)
    finally:
        runner.close()
        builder.close()


def test_attention_model_steers_a_search_on_the_gpu(hrn, tmp_path):
    """The attention cost model, fitted on the shipped points of the other cases (CPU, a few seconds), steers the search of a
    1024^3 fp16 GEMM on the real measurer; every measured kernel is verified."""
    from heron_amd.pretrain import AttentionCostModel, RecordSet
    data = RecordSet()
    data.add_tree(os.path.join(os.path.dirname(os.path.abspath(__file__)), "pretrain", "records"))
    model_path = str(tmp_path / "model.pt")
    AttentionCostModel().fit(data, None, n_epoch=25, verbose=0).save(model_path)
    env, task, runner, builder = _env(tmp_path, "CGA", 16, case=("gemm", [1024, 1024, 1024]), dtype=("float16", "float16"))
    try:
        env.config.pretrained_model = model_path
        env.config.search_generations = 2

        def ref(args):
            A, Bm = workloads.gemm_f16_inputs(1024, 1024, 1024, seed=1)
            return [A, Bm], oracle.gemm_f32(A, Bm)
        task.set_verify_func(ref, rtol=1e-2)
        env.tune("T1")
        rows = [json.loads(l) for l in open(tmp_path / "OPS" / "T1" / "records.txt")]
        assert 8 <= len(rows) <= 16 and all(row["perf"] > 0 for row in rows)
        best = math.exp(-max(row["perf"] for row in rows))
        assert 2.0 * 1024 ** 3 / best / 1e12 > 60       # sanity only: 16 trials of a random search
    finally:
        runner.close()
        builder.close()
