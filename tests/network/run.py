"""Network-level experiment:  python run.py -c configs/resnet50.json [-m trials] [-T tuned_dir]

Tunes (or re-times from earlier records) every distinct layer of a network and prints the per-layer latencies and the
estimated network latency, as tests/figure10/run.py:66-110 of the reference does.  Two sums are printed: the plain sum
over the listed layers, which is what the reference prints (run.py:105-109), and the sum weighted by each layer's
repeat count, which is what its PyTorch baselines measure (tests/figure10/pytorch/bert.py:80-85).

``-T dir`` reuses ``dir/<case>/records.txt`` of an earlier run for every case that has one (the reference's ``-t``
applies one records file to the first case only).
"""
import argparse
import json
import os
import sys

ROOT = os.path.abspath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests", "quick_start", "rocm"))

import heron_amd.runner as HeronRunner                                # noqa: E402
from heron_amd.environment import Env                                 # noqa: E402
from run import keep_best, makeConfig, run                            # noqa: E402  (tests/quick_start/rocm/run.py)


def main():
    parser = argparse.ArgumentParser(description="Tune the layers of a network and estimate its latency.")
    parser.add_argument("-p", "--platform", choices=["rocm"], default="rocm")
    parser.add_argument("-c", "--config", required=True)
    parser.add_argument("-t", "--tuned", default="", help="records.txt for the first case (reference semantics)")
    parser.add_argument("-T", "--tuned-dir", default="", help="directory with <case>/records.txt of an earlier run")
    parser.add_argument("-d", "--device_id", type=int, default=0)
    parser.add_argument("-sid", "--start_id", type=int, default=0)
    parser.add_argument("-eid", "--end_id", type=int, default=int(1e4))
    parser.add_argument("-m", "--max-trials", type=int, default=int(1e6))
    parser.add_argument("-o", "--out", default="", help="write the per-layer table as JSON")
    parser.add_argument("-v", "--verbose", action="store_true")
    parser.add_argument("--check", action="store_true", help="verify every measured kernel against a host reference")
    parser.add_argument("--incumbents", default="", metavar="DIR",
                        help="DIR/<case>/records.txt of earlier searches: their best rows are timed again in the "
                             "confirmation phase of every layer's search")
    parser.add_argument("--keep-best", default="", metavar="DIR",
                        help="after tuning a layer, write its confirmed rows and its 32 best other rows to "
                             "DIR/<case>/records.txt (the form of the files under tuned/)")
    args = parser.parse_args()

    config = makeConfig(args)
    config.max_trials = min(args.max_trials, config.max_trials)
    config.device_id = args.device_id
    config.verbose = args.verbose
    runner = HeronRunner.LocalRunner(number=config.runner_number, repeat=config.runner_repeat, min_repeat_ms=0,
                                     timeout=config.runner_timeout, device_id=args.device_id)
    option = HeronRunner.measure_option(builder=HeronRunner.LocalBuilder(timeout=config.build_timeout), runner=runner)
    keys = list(config.cases.keys())
    rows = []
    for i in range(args.start_id, min(args.end_id + 1, len(keys))):
        op_name, case, times = config.cases[keys[i]]
        config.tuned = args.tuned if i == 0 else ""
        if args.tuned_dir:
            rec = os.path.join(args.tuned_dir, keys[i], "records.txt")
            if os.path.exists(rec):
                config.tuned = rec
        print(keys[i], op_name, case, flush=True)
        inc = os.path.join(args.incumbents, keys[i], "records.txt") if args.incumbents else ""
        config.incumbents = [os.path.abspath(inc)] if inc and os.path.exists(inc) else []
        env = Env(option, config)
        tuned_here = not config.tuned
        latency = run(op_name, keys[i], case + [config.in_dtype, config.out_dtype], env, runner, args.check)
        if args.keep_best and tuned_here:
            keep_best(os.path.join(config.log_dir, "records.txt"), os.path.join(args.keep_best, keys[i], "records.txt"), 32)
        rows.append(dict(case=keys[i], op=op_name, shape=case, times=times, latency_ms=latency))
    plain = weighted = 0.0
    for r in rows:
        print("Case %s, Times : %d, latency %f ms." % (str(r["shape"]), r["times"], r["latency_ms"]))
        plain += r["latency_ms"]
        weighted += r["latency_ms"] * r["times"]
    print("Estimated network latency : ", plain)
    print("Estimated network latency weighted by layer counts : ", weighted)
    if args.out:
        with open(args.out, "w") as f:
            json.dump(dict(config=args.config, max_trials=config.max_trials, layers=rows, sum_ms=plain,
                           weighted_sum_ms=weighted), f, indent=1)
    runner.close()
    option["builder"].close()


if __name__ == "__main__":
    main()
