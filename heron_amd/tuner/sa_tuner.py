"""Simulated-annealing tuners (tuner/sa_tuner.py:13-62 of the reference).

Every member of the population takes one step per walk; a step is accepted with the Metropolis probability
exp(min((score' - score) / T, 0)) on the cost model's scores and T falls linearly to zero over the run.
(The reference computes that probability and then overwrites the decision with a plain "better score wins",
sa_tuner.py:42-44; the annealing rule is what is implemented here.)
"""
import math

import numpy as np

from .tuner import Tuner, random_walk_parallel, random_walk_sequential


class SATuner(Tuner):
    def __init__(self, config):
        super().__init__(config)
        self.t = self.config.temperature
        rounds = math.ceil(self.config.max_trials / self.config.measure_time_per_round)
        self.cool = self.t / (rounds * self.config.iter_walks + 1)

    def optimize(self, env, population, stat, s_time):
        all_samples = [] + population
        for _ in range(self.config.iter_walks):
            if hasattr(self.cost_model, "bst") and self.cost_model.bst is None:
                break
            stepped = self.walk(population, env)
            if len(stepped) == len(population):
                population = self.accept(population, stepped, self.t)
            all_samples += population
            self.t = max(self.t - self.cool, 0.0)
            self.recordStat(all_samples, env, s_time, stat)
        return population, all_samples

    def accept(self, pop, pop1, temp):
        score = np.array([x.predict for x in pop], dtype=np.float64)
        score1 = np.array([x.predict if x.valid else -np.inf for x in pop1], dtype=np.float64)
        with np.errstate(invalid="ignore", over="ignore"):
            prob = np.exp(np.minimum((score1 - score) / (temp + 1e-5), 0))
        take = np.random.random(len(pop)) < np.nan_to_num(prob, nan=0.0)
        return [pop1[i] if take[i] else pop[i] for i in range(len(pop))]

    def _walk(self, kind, env, pop, args):
        if self.config.parallel:
            samples = random_walk_parallel(kind, env.task, pop, 1, args)      # chunks come back in order
        else:
            samples = random_walk_sequential(kind, env.task, pop, 1, args)
        valid = [s for s in samples if s.valid]
        if valid:
            for s, p in zip(valid, self.predict(valid)):
                s.predict = p
        for s in samples:
            if not s.valid:
                s.predict = 0.0
        return samples


class ConstrainedRandomWalkerSATuner(SATuner):
    """Steps re-solve the CSP around the current point, so every step is feasible (sa_tuner.py:55-57)."""

    def walk(self, pop, env):
        return self._walk('constrained_random_walk', env, pop, [0.3])


class RandomWalkSATuner(SATuner):
    """Steps change one knob to a value seen feasible for it; infeasible steps are rejected (sa_tuner.py:59-61)."""

    def walk(self, pop, env):
        return self._walk('random_walk', env, pop, [self.feasible])
