"""Search-method comparison:  python run.py -c configs/gemm1024.json --methods CGA,GA,SA,CRAND [-m trials]

Tunes the same case once per search method (each into OUTS/<METHOD>/<case>/, like the per-method configs of the
reference's tests/figure12/run.sh and tests/figure13) and prints the best throughput found after 16, 32, 64, ...
measured trials, the curve tests/figure12/plot.py:11-28 draws from records.txt.  Methods: CGA (constrained GA), RCGA,
GA / SRGA / SDGA (unconstrained, stochastic-ranking and SAT-decoding GAs), IDEA, SA, CSA, CRAND (constrained random).
"""
import argparse
import json
import math
import os
import sys

ROOT = os.path.abspath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "quick_start", "rocm"))

import heron_amd.runner as HeronRunner                                # noqa: E402
from heron_amd.environment import Env                                 # noqa: E402
from run import makeConfig                                            # noqa: E402  (tests/quick_start/rocm/run.py)


def work_of(op_name, shape):
    if op_name == "gemm":
        M, K, N = shape
        return 2.0 * M * N * K
    if op_name == "bmm":
        b, M, K, N = shape
        return 2.0 * b * M * N * K
    N, H, W, CI, CO, KH, KW, s, p, d = [x for x in shape if not isinstance(x, str)][:10]
    ho = (H - ((KH - 1) * d + 1) + 2 * p) // s + 1
    wo = (W - ((KW - 1) * d + 1) + 2 * p) // s + 1
    return 2.0 * N * ho * wo * CO * KH * KW * CI


def best_so_far(records_path, work):
    curve, best = [], 0.0
    for row in open(records_path):
        perf = json.loads(row)["perf"]
        tput = work / math.exp(-perf) / 1e12 if perf else 0.0       # perf = ln(1/seconds)
        best = max(best, tput)
        curve.append(best)
    return curve


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("-p", "--platform", choices=["rocm"], default="rocm")
    ap.add_argument("-c", "--config", required=True)
    ap.add_argument("--methods", default="CGA,GA,SA,CRAND")
    ap.add_argument("-m", "--max-trials", type=int, default=int(1e6))
    ap.add_argument("-d", "--device_id", type=int, default=0)
    ap.add_argument("-o", "--out", default="summary.json")
    args = ap.parse_args()
    summary = {}
    for method in args.methods.split(","):
        config = makeConfig(args)
        config.opt_method = method
        config.out_name = os.path.join(config.out_name, method)
        config.max_trials = min(args.max_trials, config.max_trials)
        config.device_id = args.device_id
        runner = HeronRunner.LocalRunner(number=config.runner_number, repeat=config.runner_repeat, min_repeat_ms=0,
                                         timeout=config.runner_timeout, device_id=args.device_id)
        option = HeronRunner.measure_option(builder=HeronRunner.LocalBuilder(timeout=config.build_timeout), runner=runner)
        for key, (op_name, shape) in config.cases.items():
            env = Env(option, config)
            task = env.createTask(key, config.get_op(op_name), shape + [config.in_dtype, config.out_dtype], config.target_name)
            task.device_id = args.device_id
            env.tune(key)
            curve = best_so_far(os.path.join(config.log_dir, "records.txt"), work_of(op_name, shape))
            summary.setdefault(key, {})[method] = curve
        runner.close()
        option["builder"].close()
    for key, per_method in summary.items():
        marks = [n for n in (16, 32, 64, 128, 256, 512, 1024, 2048) if n <= max(len(c) for c in per_method.values())]
        print("\n%s: best T(FL)OP/s after n measured trials" % key)
        print("%-8s" % "method" + "".join("%10d" % n for n in marks) + "%10s" % "final")
        for method, curve in per_method.items():
            print("%-8s" % method + "".join("%10.1f" % curve[min(n, len(curve)) - 1] for n in marks) + "%10.1f" % curve[-1])
    with open(args.out, "w") as f:
        json.dump(summary, f)


if __name__ == "__main__":
    main()
