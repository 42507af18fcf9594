"""Writes fuzz_instances.json: template instances drawn from the tuner's own search space (constrained random
samples of the CDNA4 constraint set, fixed seed), so that the GPU parity suite also covers knob combinations nobody
picked by hand.  build() compiles them with the other shipped instances.

usage: python tests/golden/make_fuzz_instances.py
"""
import copy
import json
import os
import random
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))

import numpy as np                                                    # noqa: E402

from heron_amd import backend as B                                    # noqa: E402
from heron_amd.config import Config                                   # noqa: E402
from heron_amd.ops.rocm import getOpFromName                          # noqa: E402
from heron_amd.task.task import Task                                  # noqa: E402

TASKS = [("gemm", [2048, 1024, 2048], "float16", 8), ("gemm", [2048, 1024, 2048], "int8", 8),
         ("bmm", [8, 512, 256, 512], "float16", 4), ("c2d", [4, 28, 28, 64, 128, 3, 3, 1, 1, 1], "float16", 8),
         ("c2d", [4, 28, 28, 64, 128, 3, 3, 1, 1, 1], "int8", 6), ("c2d", [2, 30, 30, 32, 64, 3, 3, 2, 1, 1], "float16", 4),
         # few output tiles and a long K: the split-K part of the space
         ("gemm", [256, 4096, 512], "float16", 5), ("gemm", [128, 8192, 256], "int8", 5),
         ("c2d", [16, 7, 7, 512, 512, 3, 3, 1, 1, 1], "float16", 4)]
# knobs pinned for extra draws, so that rare parts of the space are always covered: (task index, knob suffix, value, count)
FORCED = [(3, "conv_window", 1, 4), (4, "conv_window", 1, 3), (0, "persistent", 1, 2), (1, "persistent", 1, 2)]


def draw(t, known, seen):
    km = copy.deepcopy(t.knob_manager)
    fixed = {}
    for suffix, value in known.items():
        name = [k for k in km.knob_names if k.endswith(suffix)][0]
        fixed[name] = value
    valid, _ = km.randSample(fixed)
    s, _ = t.instantiate(km)
    d = s.to_desc()
    tup = d.as_tuple()
    if not valid or not B.check_desc(d) or tup in seen:
        return None
    seen.add(tup)
    return {"desc": list(tup), "group_m": int(s.params["group_m"]), "split_k": int(s.params["split_k"])}


if __name__ == "__main__":
    random.seed(20240607)
    np.random.seed(20240607)
    out, seen, tasks = [], set(), []
    for op, shape, dtype, count in TASKS:
        cfg = Config()
        cfg.codegen_type = 'GPU_MFMA'
        t = Task("t", getOpFromName(op), shape + [dtype, dtype], "rocm")
        t.config = cfg
        t.make_stage_schedules()
        tasks.append(t)
    plan = [(i, {}, count) for i, (_, _, _, count) in enumerate(TASKS)]
    plan += [(i, {suffix: value}, count) for i, suffix, value, count in FORCED]
    for i, known, count in plan:
        op, shape, dtype, _ = TASKS[i]
        got = tries = 0
        while got < count and tries < 50 * count:
            tries += 1
            entry = draw(tasks[i], known, seen)
            if entry is None:
                continue
            entry["from"] = [op, shape, dtype]
            out.append(entry)
            got += 1
    with open(os.path.join(HERE, "fuzz_instances.json"), "w") as f:
        json.dump(out, f, indent=0)
    print(len(out), "instances")
