"""Runner: samples -> measure inputs -> results -> perf (runner/runner.py:9-38 of the reference)."""
import math

import numpy as np

from .measure import MeasureInput


class Runner:
    def __init__(self, measure_option):
        self.measure_option = measure_option
        self.measure_batch = None

    def results2tup(self, results):
        res = []
        for x in results:
            if x.error_no == 0:
                perf_time = np.array(x.costs).mean()
                res.append((x.error_no, math.log(1 / perf_time)))
            else:
                res.append((x.error_no, 0.0))
        return res

    def run(self, samples, perf_buffer):
        task = samples[0].task
        for sample in samples:
            assert task.name == sample.task.name
        inps = [MeasureInput(task.target, task, x.knob_manager) for x in samples]
        results = self.measure_batch(inps)
        res = self.results2tup(results)
        for idx, sample in enumerate(samples):
            error, perf = res[idx]
            sample.perf = perf
            sample.valid = error == 0
            perf_buffer.record(sample)
        best = perf_buffer.best_perf
        print('TASK %s, Cur best %f' % (task.name, best))
        for idx, sample in enumerate(samples):
            print("Sample %s" % sample.stmt_code)
            print("Perf %f , Predict %f, Prob %f" % (sample.perf, sample.predict, sample.prob))
