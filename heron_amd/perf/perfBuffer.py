"""Store of measured samples.

Interface the tuner and the cost model rely on (the reference's perf/perfBuffer.py:18-46): ``record(sample)``,
``perfs`` (sample code -> perf), ``data_x`` / ``data_y`` / ``samples`` (the successfully measured points, aligned),
``best_perf`` / ``best_sample`` and ``getPerf(sample)``.  Every new code is appended to ``<log_dir>/records.txt`` as one
JSON object per line with the reference's keys: ``code``, ``perf`` = ln(1 / seconds) (0.0 for a failed measurement),
``latency`` seconds, ``time`` (wall clock) and ``param`` (every solver variable of the sample).
"""
import json
import math
import os
import time


class perfBuffer:
    RECORD_FILE = 'records.txt'

    def __init__(self, config):
        self.config = config
        self.perfs = {}                 # code -> perf, failed measurements included (insertion-ordered)
        self.samples = []               # successfully measured samples ...
        self.data_x = []                # ... their feature vectors ...
        self.data_y = []                # ... and their perfs
        self.best_perf = None
        self.best_sample = None

    @property
    def measured_keys(self):
        return list(self.perfs)

    def record(self, sample):
        """Files one measured sample; a code seen before is ignored (the first measurement stands)."""
        code, perf = sample.stmt_code, sample.perf
        if code in self.perfs:
            return False
        self.perfs[code] = perf
        if perf != 0:
            self.samples.append(sample)
            self.data_x.append(sample.features())
            self.data_y.append(perf)
        if self.best_perf is None or perf > self.best_perf:
            self.best_perf, self.best_sample = perf, sample
        with open(os.path.join(self.config.log_dir, self.RECORD_FILE), 'a') as out:
            out.write(self.encode(sample) + '\n')
        return True

    def record_confirmed(self, sample):
        """Files the re-timing of a point at the end of a search (long repeats): one more line of records.txt, marked
        ``"confirmed": true`` - the key the reference's format does not have, and the rows ``Task.apply_best``
        prefers.  The search's own tables (``perfs``, ``data_x`` / ``data_y``) keep the first measurement."""
        self.confirmed = getattr(self, "confirmed", {})
        self.confirmed[sample.stmt_code] = sample.perf
        with open(os.path.join(self.config.log_dir, self.RECORD_FILE), 'a') as out:
            out.write(self.encode(sample, confirmed=True) + '\n')

    @staticmethod
    def encode(sample, confirmed=False):
        row = {"code": sample.stmt_code, "perf": sample.perf, "latency": math.exp(-sample.perf), "time": time.time(),
               "param": sample.knob_manager.solved_knob_vals_phenotype}
        if confirmed:
            row["confirmed"] = True
        return json.dumps(row)

    def getPerf(self, sample):
        """perf of an already measured code, None for a new one."""
        return self.perfs.get(sample.stmt_code)
