"""Constrained-random baselines (tuner/random_tuner.py:6-27 of the reference)."""
from .tuner import Tuner


class CRandTuner(Tuner):
    def check_feasible_exits(self, env, num=1e3):
        return

    def optimize(self, env, pop, stat, s_time):
        samples = [] + pop
        population = []
        for _ in range(self.config.iter_walks):
            population = self.constrained_random_sample(env, self.config.pop_num)
            samples = samples + population
            self.recordStat(samples, env, s_time, stat)
        population += sorted(samples, key=lambda x: -x.predict)[:20]
        return population, samples


class CRandSampler(Tuner):
    def check_feasible_exits(self, env, num=1e3):
        return

    def optimize(self, env, pop, stat, s_time):
        samples = [] + pop
        population = []
        for _ in range(self.config.iter_walks):
            population = self.constrained_random_sample(env, self.config.pop_num)
            samples = samples + population
            for sample in samples:
                sample.predict = 0
            self.recordStat(samples, env, s_time, stat)
        return population, samples
