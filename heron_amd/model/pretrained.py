"""Cross-task cost model: boosted trees fitted once on the measured records of OTHER tasks of the same operator.

Stands where the reference's pre-trained model does (Tuner.setPretrainedModel / run_with_pretrained,
tuner/tuner.py:32-45, fed by pretrain/): the search of a new task is steered from its first round by what earlier
tasks measured, without re-training.  The reference trains a transformer over tokenised knob names; here tasks of
one operator share their variable names, so every record's ``param`` dictionary is turned into the new task's compact
feature vector (knobs, tile and occupancy figures, the analytic estimate - ``Task.featurize``).  The target is each
record's throughput relative to the best of its own task, so tasks of different sizes can be mixed.
"""
import json
import math

import numpy as np

from ..utils import DeCode
from .cost_model import _SklearnBooster, _XgbBooster, feature_matrix, xgb


class PretrainedCostModel:
    def __init__(self, task, config):
        self.task = task
        self.bst = None
        self.num_features = None
        self.files_used = []

    def fit_from_records(self, paths, num_features):
        """``paths``: records.txt files of earlier tasks; files whose records lack one of this task's knobs (another
        operator family or an older constraint set) are skipped."""
        knobs = set(self.task.knob_manager.knob_names)
        xs, ys = [], []
        for path in paths:
            rows = [json.loads(line) for line in open(path) if line.strip()]
            rows = [r for r in rows if r["perf"] != 0]
            if not rows:
                continue
            if any(not knobs <= set(r["param"]) for r in rows):
                continue
            pts = [self.task.featurize(r["param"], own_shape=False) for r in rows]
            if any(p is None for p in pts):
                pts = [DeCode(r["code"]) for r in rows]
                if any(len(p) != num_features for p in pts):
                    continue
            best = max(r["perf"] for r in rows)
            xs += pts
            ys += [math.exp(r["perf"] - best) for r in rows]        # perf = ln(1/s): exp(diff) = relative throughput
            self.files_used.append(path)
        if not xs:
            raise ValueError("no usable records of this operator's knob set among %d files" % len(paths))
        x, y = np.array(xs, dtype=np.float64), np.array(ys, dtype=np.float64)
        self.num_features = num_features
        self.bst = _XgbBooster(x, y) if xgb is not None else _SklearnBooster(x, y)
        return len(xs)

    def predict(self, samples, output_margin=False):
        if len(samples) == 0:
            return np.zeros(0)
        return self.bst.predict(feature_matrix(samples))

    def train(self, perf_buffer):            # a pre-trained model is not re-fitted during the search
        return
