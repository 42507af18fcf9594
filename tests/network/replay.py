"""Whole-network replay:  python replay.py -c configs/resnet50.json -T tuned/resnet50 [--reps 50]

run.py times every distinct layer on its own and adds the latencies up (tests/figure10/run.py:105-109 of the
reference).  This driver answers what that sum leaves open: what the sequence costs when the layers really follow
each other on one stream.  Every layer's best record is instantiated in this process (Task.apply_best), each layer
gets its own operands, and the weighted sequence (every layer ``times`` times) is run three ways:

    isolated   sum over the sequence of each layer's own back-to-back latency (what run.py reports)
    stream     the sequence issued launch by launch on one stream, timed as a whole
    graph      the same sequence captured once into a HIP graph and replayed

The graph's result is compared with the eager one on every replay round (eager work and synchronisation between the
rounds).  Layers that need an operand adapter (the 3-channel stem) run their kernel on operands the adapter prepared once:
the replay measures kernels and their dispatch, not the Python pre-stage.
"""
import argparse
import json
import os
import sys

import numpy as np

ROOT = os.path.abspath(os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
sys.path.insert(0, ROOT)


def main():
    ap = argparse.ArgumentParser(description="Replay the tuned layers of a network as one sequence.")
    ap.add_argument("-c", "--config", required=True)
    ap.add_argument("-T", "--tuned-dir", required=True, help="directory with <case>/records.txt")
    ap.add_argument("--reps", type=int, default=50, help="timed repetitions of the whole sequence")
    ap.add_argument("--rounds", type=int, default=3, help="graph replay rounds that are checked against the eager result")
    ap.add_argument("-o", "--out", default="")
    args = ap.parse_args()

    import torch
    from heron_amd import backend as B
    from heron_amd import tuned
    if not torch.cuda.is_available():
        print("replay.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    cfg = json.load(open(args.config))["config"]
    dtype = cfg["in_dtype"]
    torch_dt = {"float16": torch.float16, "uint8": torch.uint8, "int8": torch.int8, "int32": torch.int32}
    rng = np.random.default_rng(0)
    layers = []
    for name, (op_name, shape, times) in cfg["cases"].items():
        rec = os.path.join(args.tuned_dir, name, "records.txt")
        sched, targs = tuned.instantiate(name, op_name, list(shape), dtype, rec)
        desc, prob = sched.to_desc(), sched.to_problem()
        mod = B.Module(desc)
        tens = []
        for t in targs:
            shp, dt = tuple(int(x) for x in t.shape), str(t.dtype)
            if dt == "float16":
                host = (rng.standard_normal(shp, dtype=np.float32) * 0.1).astype(np.float16)
            elif dt == "uint8":
                host = rng.integers(0, 256, shp, dtype=np.uint8)
            elif dt == "int8":
                host = rng.integers(-128, 128, shp, dtype=np.int8)
            else:
                host = np.zeros(shp, dtype=np.int32 if dt == "int32" else np.float16)
            tens.append(torch.from_numpy(host).cuda().to(torch_dt.get(dt, torch.float16)))
        layers.append(dict(name=name, mod=mod, prob=prob, a=tens[0], b=tens[1], c=tens[-1], times=int(times),
                           split=int(sched.params.get('split_k', 1))))
    launches = sum(l["times"] for l in layers)
    stream = torch.cuda.Stream()
    st = stream.cuda_stream

    def sequence():
        for l in layers:
            for _ in range(l["times"]):
                l["mod"].launch(l["prob"], l["a"].data_ptr(), l["b"].data_ptr(), l["c"].data_ptr(), st)

    # isolated latencies (also the warm-up that binds every split-K workspace before anything is captured)
    isolated = 0.0
    for l in layers:
        costs = l["mod"].time(l["prob"], l["a"].data_ptr(), l["b"].data_ptr(), l["c"].data_ptr(), number=20, repeat=5,
                              min_repeat_ms=20.0, stream=st)
        l["isolated_us"] = float(np.median(costs)) * 1e6
        isolated += l["isolated_us"] * l["times"]
    with torch.cuda.stream(stream):
        for _ in range(5):
            sequence()
        stream.synchronize()
        eager = [l["c"].clone() for l in layers]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(args.reps):
            sequence()
        e1.record(stream)
        e1.synchronize()
        stream_us = e0.elapsed_time(e1) * 1e3 / args.reps

        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            sequence()
        checked = 0
        for _ in range(args.rounds):
            for l in layers:
                l["c"].fill_(7)                      # eager work between the replays; a replay must rewrite every result
            stream.synchronize()
            graph.replay()
            stream.synchronize()
            for l, want in zip(layers, eager):
                if not torch.equal(l["c"], want):
                    print("graph replay differs from the eager result in %s" % l["name"], file=sys.stderr)
                    sys.exit(1)
            checked += 1
        e0.record(stream)
        for _ in range(args.reps):
            graph.replay()
        e1.record(stream)
        e1.synchronize()
        graph_us = e0.elapsed_time(e1) * 1e3 / args.reps
    out = dict(config=args.config, layers=len(layers), launches=launches, kernel_launches=launches + sum(
                   l["times"] for l in layers if l["split"] > 1),
               isolated_sum_us=isolated, stream_us=stream_us, graph_us=graph_us, graph_rounds_checked=checked,
               per_launch_us=dict(isolated=isolated / launches, stream=stream_us / launches, graph=graph_us / launches))
    print("%d layers, %d launches per pass" % (len(layers), launches))
    print("isolated sum %.1f us | one stream %.1f us | HIP graph %.1f us (%d replay rounds equal to eager)"
          % (isolated, stream_us, graph_us, checked))
    print(json.dumps(out))
    if args.out:
        with open(args.out, "w") as f:
            json.dump(dict(out, per_layer=[dict(case=l["name"], times=l["times"], isolated_us=l["isolated_us"])
                                           for l in layers]), f, indent=1)
    for l in layers:
        l["mod"].close()


if __name__ == "__main__":
    main()
