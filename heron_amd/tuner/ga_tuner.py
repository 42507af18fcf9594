"""Genetic tuners (tuner/ga_tuner.py:13-110 of the reference).

CGATuner is the constrained genetic algorithm: each walk draws a random 20 % of *all* CSP variables
as key variables, roulette-selects parents, and creates every child by solving the CSP with each key
variable restricted to one of its two parents' values (one key left free as the mutation), so every
child is feasible by construction.
"""
import os
import random

import numpy as np

from ..multi import Job
from ..sample import Sample
from ..utils import Code, anaCostModel
from .tuner import Tuner, _run_jobs


class GATuner(Tuner):
    def optimize(self, env, population, stat, s_time):
        all_pop = [] + population
        for _ in range(self.config.iter_walks):
            # nothing measured yet: the reference has no fitness to evolve on (ga_tuner.py:16-17); with an analytic
            # estimate of the template the walks evolve on that, so the first measured batch is already a good one
            if hasattr(self.cost_model, 'bst') and self.cost_model.bst is None and \
                    not getattr(self.cost_model, 'has_prior', False):
                break
            self.inferKeyVariables(env, population)
            population = self.RankPop(population)
            population = self.Selection(population, self.config.select_num)
            population = self.crossoverAndMutate(population, env.task)
            all_pop += population
            self.recordStat(all_pop, env, s_time, stat)
            prevs = sorted(all_pop, key=lambda x: x.predict)[-20:]
            population = population + prevs
        self.removeInvalid(all_pop)
        return population, all_pop

    def inferKeyVariables(self, env, pop):
        return

    def RankPop(self, pop):
        return pop

    def Selection(self, pop, num):
        return self.RouletteWheelSelection(pop, num)

    def removeInvalid(self, all_pop):
        for sample in all_pop:
            if not sample.valid:
                sample.predict = 0.0

    def crossoverAndMutate(self, samples, task):
        if self.config.parallel:
            res = crossoverAndMutateParallel('Unconstrained', self.config.pop_num, samples, task,
                                             self.config.parallel_num, self.feasible)
        else:
            res = crossoverAndMutateSequential('Unconstrained', self.config.pop_num, samples, task, self.feasible)
        vsamples = [s for s in res if s.valid]
        if vsamples != []:
            perfs = self.predict(vsamples)
            for idx, sample in enumerate(vsamples):
                sample.predict = perfs[idx]
        for sample in res:
            if not sample.valid:
                sample.predict = 0
        return res


class CGATuner(GATuner):
    def __init__(self, config):
        super().__init__(config)
        # the last quarter of the measuring rounds refines the incumbents knob by knob: the fine knobs (issue order,
        # load spread, raster group, epilogue kind) move a good tile by a few percent, less than the cost model resolves
        self.refine_share = float(getattr(config, 'refine_share', 0.25))

    def check_feasible_exits(self, env, num=1e3):
        return

    def inferKeyVariables(self, env, pop):
        vars_ = list(env.task.knob_manager.solver.vals.keys())
        random.shuffle(vars_)
        self.key_variables = vars_[:int(self.config.crossover_key_ratio * len(vars_))]

    def crossoverAndMutate(self, samples, task):
        if hasattr(self, "key_variables") and self.key_variables is not None:
            keys = self.key_variables
        else:
            keys = anaCostModel(self.cost_model, list(task.knob_manager.solver.vals.keys()))
            keys = keys[:int(self.config.crossover_key_ratio * len(keys))]
        if self.config.parallel:
            res = crossoverAndMutateParallel('Constrained', self.config.pop_num, samples, task,
                                             self.config.parallel_num, keys)
        else:
            res = crossoverAndMutateSequential('Constrained', self.config.pop_num, samples, task, keys)
        perfs = self.predict(res)
        for idx, sample in enumerate(res):
            sample.predict = perfs[idx]
        return res


class RCGATuner(GATuner):
    """CGA with fresh random key variables per call (ga_tuner.py:94-110)."""

    def check_feasible_exits(self, env, num=1e3):
        return

    def crossoverAndMutate(self, samples, task):
        keys = list(task.knob_manager.solver.vals.keys())
        random.shuffle(keys)
        keys = keys[:int(self.config.crossover_key_ratio * len(keys))]
        if self.config.parallel:
            res = crossoverAndMutateParallel('Constrained', self.config.pop_num, samples, task,
                                             self.config.parallel_num, keys)
        else:
            res = crossoverAndMutateSequential('Constrained', self.config.pop_num, samples, task, keys)
        perfs = self.predict(res)
        for idx, sample in enumerate(res):
            sample.predict = perfs[idx]
        return res


class SRGATuner(GATuner):
    """GA over all variables without constraint handling in the operators; constraint pressure comes from
    stochastic ranking: a bubble sort whose comparisons use the predicted score when both neighbours are feasible
    or with probability ``pf``, and the total violation otherwise (ga_tuner.py:113-154)."""
    SWEEPS, PF = 10, 0.45

    def Selection(self, pop, num):
        return self.RankSelection(pop, num)

    def RankPop(self, pop):
        order = list(pop)
        for _ in range(self.SWEEPS):
            swapped = False
            for j in range(len(order) - 1):
                a, b = order[j], order[j + 1]
                va, vb = a.violation or 0, b.violation or 0
                if (va == 0 and vb == 0) or random.random() < self.PF:
                    out_of_order = a.predict < b.predict
                else:
                    out_of_order = va > vb
                if out_of_order:
                    order[j], order[j + 1] = b, a
                    swapped = True
            if not swapped:
                break
        return order

    def crossoverAndMutate(self, samples, task):
        res = _offspring(self.config, 'UnconstrainedAll', samples, task, self.feasible)
        perfs = self.predict(res)
        for idx, sample in enumerate(res):
            sample.predict = perfs[idx]
        return res


class SDGATuner(GATuner):
    """GA whose genotype is decoded into a feasible phenotype by repairing it with the solver
    (SAT-decoding, ga_tuner.py:157-166)."""

    def crossoverAndMutate(self, samples, task):
        res = _offspring(self.config, 'SATDecoding', samples, task, self.feasible)
        perfs = self.predict(res)
        for idx, sample in enumerate(res):
            sample.predict = perfs[idx]
        return res


def _offspring(config, kind, samples, task, extra):
    if config.parallel:
        return crossoverAndMutateParallel(kind, config.pop_num, samples, task, config.parallel_num, extra)
    return crossoverAndMutateSequential(kind, config.pop_num, samples, task, extra)


def crossoverAndMutateParallel(kind, number, population, task, parallel_num, extra, timeout=60):
    work_load = int((number + parallel_num - 1) // parallel_num)
    jobs = [Job(crossoverAndMutateSequential, (kind, work_load, population, task, extra), timeout)
            for _ in range(parallel_num)]
    return _run_jobs(jobs)


def crossoverAndMutateSequential(kind, number, population, task, extra):
    random.seed(int.from_bytes(os.urandom(8), "little"))
    np.random.seed(int.from_bytes(os.urandom(4), "little"))
    ret = []
    if len(population) == 0:
        return ret
    for _ in range(number):
        m1 = population[random.randint(0, len(population) - 1)]
        m2 = population[random.randint(0, len(population) - 1)]
        child = Sample(task)
        if kind == 'Constrained':
            point, valid = child.knob_manager.constrained_crossover_and_mutate(m1.knob_manager, m2.knob_manager, extra)
        elif kind == 'UnconstrainedAll':
            point, valid, child.violation = child.knob_manager.crossover_and_mutate_all(m1.knob_manager, m2.knob_manager, extra)
        elif kind == 'SATDecoding':
            point, valid = child.knob_manager.satdecoding_crossover_and_mutate(m1.knob_manager, m2.knob_manager, extra)
        elif kind == 'SBX':
            point, valid, child.violations = child.knob_manager.SBX_crossover_and_mutation(m1.knob_manager, m2.knob_manager, extra)
        else:
            point, valid = child.knob_manager.crossover_and_mutate(m1.knob_manager, m2.knob_manager, extra)
        child.point = point
        child.valid = bool(valid)
        child.stmt_code = Code(list(point))
        ret.append(child)
    return ret
