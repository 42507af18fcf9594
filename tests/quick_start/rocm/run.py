"""Tune and time cases on MI355X:  python run.py -p rocm -c quick_start.json

Same command line, JSON schema, output files (<out_name>/<case>/{schedule.py, constraints.py,
records.txt, stat.txt}) and final ``PASS`` / ``Case ..., latency ... ms.`` lines as the reference's
tests/quick_start/{dlboost,tensorcore}/run.py:19-110, with ``-p rocm`` selecting the MFMA operator
set, the CDNA4 constraint set and the HIP measurer.  ``--check`` additionally verifies every
measured kernel against a numpy host reference (Task.set_verify_func).
"""
import argparse
import os
import sys

import numpy as np

ROOT = os.path.abspath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "..", ".."))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import heron_amd.ops.rocm as heron_rocm                              # noqa: E402
import heron_amd.runner as HeronRunner                                # noqa: E402
from heron_amd.config import configFromFile                           # noqa: E402
from heron_amd.environment import Env                                 # noqa: E402
from heron_amd import workloads                                       # noqa: E402


def makeConfig(args):
    config = configFromFile(args.config)
    if args.platform == "rocm":
        config.target_name = 'rocm'
        config.codegen_type = 'GPU_MFMA'
        config.get_op = heron_rocm.getOpFromName
    return config


def _im2col(X, KH, KW, stride, pad, dil):
    N, H, W, CI = X.shape
    HO = (H - ((KH - 1) * dil + 1) + 2 * pad) // stride + 1
    WO = (W - ((KW - 1) * dil + 1) + 2 * pad) // stride + 1
    P = np.zeros((N, H + 2 * pad, W + 2 * pad, CI), X.dtype)
    P[:, pad:pad + H, pad:pad + W, :] = X
    cols = np.empty((N, HO, WO, KH, KW, CI), X.dtype)
    for ry in range(KH):
        for rx in range(KW):
            cols[:, :, :, ry, rx, :] = P[:, ry * dil:ry * dil + (HO - 1) * stride + 1:stride,
                                         rx * dil:rx * dil + (WO - 1) * stride + 1:stride, :]
    return cols.reshape(N * HO * WO, KH * KW * CI), (N, HO, WO)


def host_reference(op_name):
    """numpy reference for --check: returns func(params) -> ([inputs], expected_output)."""
    def ref(params):
        shape = [x for x in params[:-2] if not isinstance(x, str)]     # drop a w_format entry
        f16 = params[-2] == "float16"
        wide = np.float32 if f16 else np.int64
        if op_name == "gemm":
            M, K, N = shape
            A, B = workloads.gemm_f16_inputs(M, K, N) if f16 else workloads.gemm_u8s8_inputs(M, K, N)
            return [A, B], A.astype(wide) @ B.astype(wide).T
        if op_name == "bmm":
            b, M, K, N = shape
            if f16:
                A, B = workloads.bmm_qk_inputs(b, M, K, N)
            else:
                A, B = (np.stack(t) for t in zip(*[workloads.gemm_u8s8_inputs(M, K, N, seed=i) for i in range(b)]))
            return [A, B], np.einsum("bik,bjk->bij", A.astype(wide), B.astype(wide))
        N, H, W, CI, CO, KH, KW, stride, pad, dil = shape
        X, Wt = (workloads.conv2d_inputs if f16 else workloads.conv2d_u8s8_inputs)(N, H, W, CI, CO, KH, KW)
        cols, oshape = _im2col(X.astype(wide), KH, KW, stride, pad, dil)
        return [X, Wt], (cols @ Wt.astype(wide).reshape(CO, -1).T).reshape(*oshape, CO)
    return ref


def keep_best(src, dst, n):
    """Writes the rows of a search that are worth keeping to ``dst`` (what ``-t`` and the benchmark later load through
    Task.apply_best): the ``n`` best rows re-timed by the confirmation phase and the ``n`` best of the others, failed
    measurements dropped."""
    import json
    rows = [json.loads(line) for line in open(src) if line.strip()]
    confirmed = sorted((r for r in rows if r.get("confirmed") and r["perf"] > 0), key=lambda r: -r["perf"])[:n]
    plain = sorted((r for r in rows if not r.get("confirmed") and r["perf"] > 0), key=lambda r: -r["perf"])[:n]
    os.makedirs(os.path.dirname(os.path.abspath(dst)), exist_ok=True)
    with open(dst, "w") as out:
        for r in plain + sorted(confirmed, key=lambda r: r["perf"]):          # the best confirmed row comes last
            out.write(json.dumps(r) + "\n")
    return len(plain) + len(confirmed)


def run(op_name, task_name, params, env, runner, check=False):
    config = env.config
    op = config.get_op(op_name)
    task = env.createTask(task_name, op, params, config.target_name)
    task.device_id = config.device_id
    if check and op_name in ("gemm", "bmm", "c2d", "c2d_nhwc"):
        task.set_verify_func(host_reference(op_name), rtol=1e-2)
    if config.tuned == "":
        env.tune(task_name)
        config.tuned = os.path.join(config.log_dir, 'records.txt')
    s, args = task.apply_best(config.tuned)
    print("Best instance:", s.describe())
    latency = runner.time_instance(s, args, number=config.runner_number, repeat=config.runner_repeat,
                                   min_repeat_ms=500, cold=getattr(config, "cold", False)) * 1e3
    if latency > 0:
        print("PASS")
    return latency


if __name__ == '__main__':
    parser = argparse.ArgumentParser(description='Run cases in Heron.')
    parser.add_argument("-p", "--platform", choices=['rocm'], type=str, default="rocm",
                        help="Hardware platform: rocm (MI355X, MFMA templates).")
    parser.add_argument("-c", "--config", type=str, required=True,
                        help="Config file name: describes the param of test_cases")
    parser.add_argument("-t", "--tuned", type=str, default="",
                        help="records.txt of an earlier run: tuned parameters for direct use.")
    parser.add_argument("-d", "--device_id", type=int, default=0, help="Device index for measurement")
    parser.add_argument("-sid", "--start_id", type=int, default=0, help="Start case number in test cases")
    parser.add_argument("-eid", "--end_id", type=int, default=int(1e4), help="End case number in test cases")
    parser.add_argument("-v", "--verbose", action="store_true", help="Show some information if enabled.")
    parser.add_argument("-m", "--max-trials", type=int, default=int(1e6), help="Max trials by command line")
    parser.add_argument("--check", action="store_true", help="verify measured kernels against a host reference")
    parser.add_argument("--cold", action="store_true",
                        help="time every launch from flushed caches (the runner's enable_cpu_cache_flush of "
                             "tests/quick_start/dlboost/run.py:89-96, on the GPU): for cases bound by HBM traffic")
    parser.add_argument("--keep-best", type=str, default="", metavar="DIR",
                        help="after tuning a case, copy its confirmed rows and its 32 best other rows to "
                             "DIR/<case>/records.txt (the form of the files under tuned/)")
    parser.add_argument("--incumbents", type=str, default="", metavar="DIR",
                        help="DIR/<case>/records.txt of earlier searches (the layout --keep-best writes): their best rows "
                             "are timed again in the confirmation phase, beside this search's own best tiles")
    parser.add_argument("--pretrained-model", type=str, default="",
                        help="attention cost model saved by tests/pretrain/train_model.py: the search is steered by it "
                             "from the first round and it is not re-trained (pretrain/tune_with_pretrained.py)")
    parser.add_argument("--pretrained", type=str, default="",
                        help="comma separated records.txt files of earlier tasks of the same operator: steer the search "
                             "with a cost model fitted on them instead of training one from scratch")
    args = parser.parse_args()
    print("Heron device ", args.device_id)

    config = makeConfig(args)
    config.max_trials = min(args.max_trials, config.max_trials)
    config.device_id = args.device_id
    config.tuned = args.tuned
    config.verbose = args.verbose
    config.pretrained_records = [p for p in args.pretrained.split(",") if p]
    config.pretrained_model = os.path.abspath(args.pretrained_model) if args.pretrained_model else ""
    config.cold = args.cold
    runner = HeronRunner.LocalRunner(number=config.runner_number, repeat=config.runner_repeat, min_repeat_ms=0,
                                     timeout=config.runner_timeout, enable_cpu_cache_flush=args.cold,
                                     device_id=args.device_id)
    measure_option = HeronRunner.measure_option(
        builder=HeronRunner.LocalBuilder(timeout=config.build_timeout),
        runner=runner,
    )
    cases = []
    case_keys = list(config.cases.keys())
    for i in range(args.start_id, min(args.end_id + 1, len(case_keys))):
        if i >= 1:
            config.tuned = ''
        op_name, case = config.cases[case_keys[i]]
        print(case)
        if args.incumbents:
            config.incumbents = [os.path.abspath(os.path.join(args.incumbents, case_keys[i], 'records.txt'))]
        env = Env(measure_option, config)
        latency = run(op_name, case_keys[i], case + [config.in_dtype, config.out_dtype], env, runner, args.check)
        cases.append([case, latency])
        if args.keep_best and not args.tuned:
            kept = keep_best(os.path.join(config.log_dir, 'records.txt'),
                             os.path.join(args.keep_best, case_keys[i], 'records.txt'), 32)
            print("kept %d rows of %s under %s" % (kept, case_keys[i], args.keep_best))
    for tup in cases:
        print("Case %s, latency %f ms." % (str(tup[0]), tup[1]))
    runner.close()
    measure_option["builder"].close()
