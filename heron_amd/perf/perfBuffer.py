"""Measured results: de-duplicated by sample code, appended to records.txt as JSON lines
``{"code","perf","latency","time","param"}`` (perf/perfBuffer.py:18-46 of the reference);
``perf`` is ln(1/seconds), ``latency`` seconds."""
import json
import math
import os
import time


class perfBuffer:
    def __init__(self, config):
        self.perfs = {}
        self.data_x = []
        self.data_y = []
        self.samples = []
        self.measured_keys = []
        self.best_perf = None
        self.best_sample = None
        self.config = config

    def record(self, sample):
        perf = sample.perf
        code = sample.stmt_code
        if code in self.measured_keys:
            return
        self.measured_keys.append(code)
        self.perfs[code] = perf
        if perf != 0:
            self.samples.append(sample)
            self.data_x.append(sample.point)
            self.data_y.append(perf)
        if self.best_perf is None or perf > self.best_perf:
            self.best_perf = perf
            self.best_sample = sample
        with open(os.path.join(self.config.log_dir, 'records.txt'), 'a') as f:
            f.write(self.encode(sample) + '\n')

    def encode(self, sample):
        return json.dumps({
            "code": sample.stmt_code,
            "perf": sample.perf,
            "latency": math.exp(-sample.perf),
            "time": time.time(),
            "param": sample.knob_manager.solved_knob_vals_phenotype,
        })

    def getPerf(self, task):
        code = task.stmt_code
        if code not in self.measured_keys:
            return None
        return self.perfs.get(code, 0.0)
