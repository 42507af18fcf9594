"""The tuned template instances of the benchmark configurations.

``tests/quick_start/rocm/tuned/<CASE>/records.txt`` holds the best records of a search on MI355X per case
(``run.py -c configs/<case>.json --keep-best N``); ``load(name)`` replays the best of them through
``Task.apply_best`` - the same path ``run.py -t`` takes - and returns the template descriptor, its launch-time
parameters and the record it came from.  The benchmark, smoke and the full-size GPU tests all run these instances.
"""
import contextlib
import io
import json
import math
import os
from collections import namedtuple

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TUNED_DIR = os.path.join(ROOT, "tests", "quick_start", "rocm", "tuned")

# name -> (records directory, operator, shape arguments, element type)
CASES = {
    "gemm_u8s8_8192": ("GEMM_INT8/G8192", "gemm", [8192, 8192, 8192], "int8"),
    "gemm_f16_8192": ("GEMM_F16_8192/G8192", "gemm", [8192, 8192, 8192], "float16"),
    "gemm_f16_4096": ("GEMM_F16_4096/G4096", "gemm", [4096, 4096, 4096], "float16"),
    "bmm_f16_qk": ("BMM_F16/QK", "bmm", [192, 512, 64, 512], "float16"),
    "bmm_f16_pv": ("BMM_F16/PV", "bmm", [192, 512, 512, 64], "float16"),
    "conv2d_f16_resnet": ("C2D_F16/C1", "c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1], "float16"),
    "conv2d_u8s8_resnet": ("C2D_INT8/C1", "c2d", [32, 56, 56, 64, 64, 3, 3, 1, 1, 1, "OhwI64o4i"], "int8"),
}

TunedInstance = namedtuple("TunedInstance", "name desc group_m split_k code search_latency records params")

_cache = {}


def records_path(name):
    return os.path.join(TUNED_DIR, CASES[name][0], "records.txt")


def instantiate(name, op, shape, dtype, path):
    """(template schedule, kernel-side argument tensors) of the best record in ``path`` for one case."""
    from .config import Config
    from .ops.rocm import getOpFromName
    from .task.task import Task
    cfg = Config()
    cfg.codegen_type, cfg.target_name = 'GPU_MFMA', 'rocm'
    task = Task(name, getOpFromName(op), list(shape) + [dtype, dtype], "rocm")
    task.config = cfg
    with contextlib.redirect_stdout(io.StringIO()):      # building the template prints the task's arguments
        return task.apply_best(path)


def case_file_descs(config_path, tuned_dir):
    """Descriptors of the best record of every case of a JSON case file that has ``tuned_dir/<case>/records.txt``
    (the layers of a network, tests/network/configs + tests/network/tuned)."""
    cfg = json.load(open(config_path))["config"]
    out = []
    for name, entry in cfg["cases"].items():
        path = os.path.join(tuned_dir, name, "records.txt")
        if os.path.exists(path):
            out.append(instantiate(name, entry[0], entry[1], cfg["in_dtype"], path)[0].to_desc())
    return out


def load(name):
    """The best record of case ``name`` as a TunedInstance (cached)."""
    if name in _cache:
        return _cache[name]
    from .task.task import Task
    rel, op, shape, dtype = CASES[name]
    path = records_path(name)
    sched, _ = instantiate(name, op, shape, dtype, path)
    best = Task.best_record(path)
    inst = TunedInstance(name, sched.to_desc(), int(sched.params['group_m']), int(sched.params.get('split_k', 1)),
                         best["code"], math.exp(-best["perf"]), path, dict(sched.params))
    _cache[name] = inst
    return inst


def all_descs():
    """Descriptors of every tuned case (what build() precompiles)."""
    return [load(name).desc for name in CASES]
