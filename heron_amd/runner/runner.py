"""Turns a batch of samples into measurements: one MeasureInput per sample through the measure option's
``measure_batch``, perf = ln(1 / mean seconds) for a clean result and 0.0 for any error number, every sample filed
in the perf buffer.  Same role and printed lines as the reference's runner/runner.py:9-38."""
import math

import numpy as np

from .measure import MeasureInput


def perf_of(result):
    """(ok, perf) of one MeasureResult."""
    if result.error_no != 0:
        return False, 0.0
    return True, math.log(1.0 / float(np.mean(result.costs)))


class Runner:
    def __init__(self, measure_option):
        self.measure_option = measure_option
        self.measure_batch = None           # set by Env once the task is known

    def results2tup(self, results):
        return [(r.error_no, perf_of(r)[1]) for r in results]

    def run(self, samples, perf_buffer):
        if not samples:
            return
        task = samples[0].task
        if any(s.task.name != task.name for s in samples):
            raise ValueError("a measurement batch must belong to one task")
        results = self.measure_batch([MeasureInput(task.target, task, s.knob_manager) for s in samples])
        for sample, result in zip(samples, results):
            sample.valid, sample.perf = perf_of(result)
            perf_buffer.record(sample)
        print('TASK %s, Cur best %f' % (task.name, perf_buffer.best_perf))
        for sample in samples:
            print("Sample %s" % sample.stmt_code)
            print("Perf %f , Predict %f, Prob %f" % (sample.perf, sample.predict, sample.prob))
