"""Baselines without a search operator: every walk draws a fresh batch of constrained-random samples.

``CRandTuner`` lets the cost model rank what it drew (the batch plus the 20 best-predicted points seen so far go on to
selection); ``CRandSampler`` ignores the model altogether (all predictions zeroed), i.e. pure constrained-random
search.  Same roles as the two classes of the reference's tuner/random_tuner.py:6-27."""
from .tuner import Tuner


class _ConstrainedRandom(Tuner):
    use_model = True

    def check_feasible_exits(self, env, num=1e3):
        return              # constrained sampling needs no per-knob feasible sets

    def optimize(self, env, pop, stat, s_time):
        seen = list(pop)
        batch = []
        for _ in range(self.config.iter_walks):
            batch = self.constrained_random_sample(env, self.config.pop_num)
            seen += batch
            if not self.use_model:
                for sample in seen:
                    sample.predict = 0
            self.recordStat(seen, env, s_time, stat)
        if self.use_model:
            batch = batch + sorted(seen, key=lambda s: s.predict, reverse=True)[:20]
        return batch, seen


class CRandTuner(_ConstrainedRandom):
    use_model = True


class CRandSampler(_ConstrainedRandom):
    use_model = False
