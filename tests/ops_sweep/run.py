"""Per-operator experiment:  python run.py [-m trials] [--only f16_gemm,int8_c2d] [--configs DIR] [--check] [-o results.json]

Tunes every case of every configs/*.json (the operator shape lists of the reference's tests/figure6 and tests/figure8
experiments) with the rocm backend and writes one table of latencies; each config can also be run on its own with
tests/quick_start/rocm/run.py.
"""
import argparse
import glob
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.abspath(os.path.join(HERE, "..", ".."))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "quick_start", "rocm"))

import heron_amd.runner as HeronRunner                                # noqa: E402
from heron_amd.environment import Env                                 # noqa: E402
from run import makeConfig, run                                       # noqa: E402  (tests/quick_start/rocm/run.py)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("-p", "--platform", choices=["rocm"], default="rocm")
    ap.add_argument("-m", "--max-trials", type=int, default=int(1e6))
    ap.add_argument("-d", "--device_id", type=int, default=0)
    ap.add_argument("--only", default="", help="comma separated config names without .json")
    ap.add_argument("-o", "--out", default="results.json")
    ap.add_argument("--configs", default=os.path.join(HERE, "configs"), help="directory of case files (default: the shipped lists)")
    ap.add_argument("--check", action="store_true", help="verify every measured kernel against a host reference "
                                                         "(gemm, bmm and c2d cases; the measurer reports a mismatch as error 100)")
    args = ap.parse_args()
    names = sorted(os.path.basename(f)[:-5] for f in glob.glob(os.path.join(args.configs, "*.json")))
    if args.only:
        names = [n for n in names if n in args.only.split(",")]
    rows = []
    for name in names:
        args.config = os.path.join(args.configs, name + ".json")
        config = makeConfig(args)
        config.max_trials = min(args.max_trials, config.max_trials)
        config.device_id = args.device_id
        runner = HeronRunner.LocalRunner(number=config.runner_number, repeat=config.runner_repeat, min_repeat_ms=0,
                                         timeout=config.runner_timeout, device_id=args.device_id)
        option = HeronRunner.measure_option(builder=HeronRunner.LocalBuilder(timeout=config.build_timeout), runner=runner)
        for key, (op_name, shape) in config.cases.items():
            config.tuned = ""
            env = Env(option, config)
            print(name, key, op_name, shape, flush=True)
            latency = run(op_name, key, shape + [config.in_dtype, config.out_dtype], env, runner, args.check)
            rows.append(dict(config=name, case=key, op=op_name, shape=shape, dtype=config.in_dtype, latency_ms=latency))
            with open(args.out, "w") as f:
                json.dump(rows, f, indent=1)
        runner.close()
        option["builder"].close()
    for r in rows:
        print("%-10s %-6s %-56s %.5f ms" % (r["config"], r["case"], r["shape"], r["latency_ms"]))


if __name__ == "__main__":
    main()
