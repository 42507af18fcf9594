"""Genetic tuners (the family of tuner/ga_tuner.py:13-166 of the reference).

All of them share one generation step: pick the key variables, order and select parents, breed ``pop_num`` children,
score them, keep the 20 best seen so far in the breeding pool.  The tuners differ in how a child is made from two
parents (``BREED``) and in how parents are ranked and selected:

* ``GA``    one-point crossover + one mutated knob, validated afterwards (children may be infeasible);
* ``CGA``   constrained: a random 20 % of *all* CSP variables are key variables, and a child is the solver's answer to
            "each key variable equals one of its two parents' values, one key left free" - feasible by construction;
* ``RCGA``  CGA with fresh key variables for every breeding call;
* ``SRGA``  unconstrained operators over all variables, stochastic ranking against the violation;
* ``SDGA``  the crossed genotype is repaired into a feasible phenotype by the solver (SAT decoding).
"""
import os
import random

import numpy as np

from ..multi import Job
from ..sample import Sample
from ..utils import Code, anaCostModel
from .tuner import Tuner, _run_jobs

KEEP_BEST = 20          # best individuals seen in this call that rejoin the breeding pool after every generation


# ---------------------------------------------------------------------------------------------- making children
def _child_unconstrained(km, a, b, extra):
    point, valid = km.crossover_and_mutate(a, b, extra)
    return point, valid, {}


def _child_constrained(km, a, b, keys):
    point, valid = km.constrained_crossover_and_mutate(a, b, keys)
    return point, valid, {}


def _child_all_variables(km, a, b, feasible):
    point, valid, violation = km.crossover_and_mutate_all(a, b, feasible)
    return point, valid, {'violation': violation}


def _child_sat_decoding(km, a, b, feasible):
    point, valid = km.satdecoding_crossover_and_mutate(a, b, feasible)
    return point, valid, {}


def _child_sbx(km, a, b, feasible):
    point, valid, violations = km.SBX_crossover_and_mutation(a, b, feasible)
    return point, valid, {'violations': violations}


BREED = {'Unconstrained': _child_unconstrained, 'Constrained': _child_constrained,
         'UnconstrainedAll': _child_all_variables, 'SATDecoding': _child_sat_decoding, 'SBX': _child_sbx}


def crossoverAndMutateSequential(kind, number, population, task, extra):
    """``number`` children of random parent pairs (runs inside a forked worker when the tuner samples in parallel)."""
    random.seed(int.from_bytes(os.urandom(8), "little"))
    np.random.seed(int.from_bytes(os.urandom(4), "little"))
    make = BREED[kind]
    children = []
    for _ in range(number if population else 0):
        mother, father = random.choice(population), random.choice(population)
        child = Sample(task)
        point, valid, attrs = make(child.knob_manager, mother.knob_manager, father.knob_manager, extra)
        for name, value in attrs.items():
            setattr(child, name, value)
        child.point, child.valid, child.stmt_code = point, bool(valid), Code(list(point))
        children.append(child)
    return children


def crossoverAndMutateParallel(kind, number, population, task, parallel_num, extra, timeout=60):
    share = -(-number // parallel_num)
    return _run_jobs([Job(crossoverAndMutateSequential, (kind, share, population, task, extra), timeout)
                      for _ in range(parallel_num)])


def _offspring(config, kind, samples, task, extra):
    if config.parallel:
        return crossoverAndMutateParallel(kind, config.pop_num, samples, task, config.parallel_num, extra)
    return crossoverAndMutateSequential(kind, config.pop_num, samples, task, extra)


# ---------------------------------------------------------------------------------------------------- the tuners
class GATuner(Tuner):
    KIND = 'Unconstrained'

    def optimize(self, env, population, stat, s_time):
        seen = list(population)
        for _ in range(self.config.iter_walks):
            if not self._has_fitness():
                break
            self.inferKeyVariables(env, population)
            parents = self.Selection(self.RankPop(population), self.config.select_num)
            population = self.crossoverAndMutate(parents, env.task)
            seen += population
            self.recordStat(seen, env, s_time, stat)
            population = population + sorted(seen, key=lambda x: x.predict)[-KEEP_BEST:]
        self.removeInvalid(seen)
        return population, seen

    def _has_fitness(self):
        """Nothing measured yet: the reference has no fitness to evolve on and skips the walks (ga_tuner.py:16-17).
        With an analytic estimate of the template the walks evolve on that, so the first measured batch is a good one."""
        model = self.cost_model
        untrained = hasattr(model, 'bst') and model.bst is None
        return not untrained or getattr(model, 'has_prior', False)

    # hooks of the generation step
    def inferKeyVariables(self, env, pop):
        return

    def RankPop(self, pop):
        return pop

    def Selection(self, pop, num):
        return self.RouletteWheelSelection(pop, num)

    def breeding_extra(self, task):
        return self.feasible

    def removeInvalid(self, all_pop):
        for sample in all_pop:
            if not sample.valid:
                sample.predict = 0.0

    def _score(self, children):
        """Predicted score for the feasible children, zero for the others."""
        good = [c for c in children if c.valid]
        for child, p in zip(good, self.predict(good) if good else []):
            child.predict = p
        for child in children:
            if not child.valid:
                child.predict = 0
        return children

    def crossoverAndMutate(self, samples, task):
        return self._score(_offspring(self.config, self.KIND, samples, task, self.breeding_extra(task)))


class _ConstrainedGA(GATuner):
    """Children come out of the solver, so every one of them is feasible and no feasible-value table is needed."""
    KIND = 'Constrained'

    def check_feasible_exits(self, env, num=1e3):
        return

    def _random_keys(self, task):
        names = list(task.knob_manager.solver.vals.keys())
        random.shuffle(names)
        return names[:int(self.config.crossover_key_ratio * len(names))]

    def _score(self, children):
        for child, p in zip(children, self.predict(children) if children else []):
            child.predict = p
        return children


class CGATuner(_ConstrainedGA):
    def __init__(self, config):
        super().__init__(config)
        self.key_variables = None

    def refinement_share(self):
        # the last quarter of the measuring rounds refines the incumbents knob by knob: the fine knobs (issue order,
        # load spread, raster group, epilogue kind) move a good tile by a few percent, less than the cost model resolves
        return float(getattr(self.config, 'refine_share', 0.25))

    def confirmation_tiles(self):
        return int(getattr(self.config, 'confirm_tiles', 8))

    def inferKeyVariables(self, env, pop):
        self.key_variables = self._random_keys(env.task)

    def breeding_extra(self, task):
        if self.key_variables is not None:
            return self.key_variables
        # no generation step has run yet: the variables the cost model weighs most (ga_tuner.py:79-83)
        ranked = anaCostModel(self.cost_model, list(task.knob_manager.solver.vals.keys()))
        return ranked[:int(self.config.crossover_key_ratio * len(ranked))]


class RCGATuner(_ConstrainedGA):
    """CGA with fresh random key variables per breeding call (ga_tuner.py:94-110)."""

    def breeding_extra(self, task):
        return self._random_keys(task)


class SRGATuner(GATuner):
    """GA over all variables without constraint handling in the operators; constraint pressure comes from
    stochastic ranking: a bubble sort whose comparisons use the predicted score when both neighbours are feasible
    or with probability ``PF``, and the total violation otherwise (ga_tuner.py:113-154)."""
    KIND = 'UnconstrainedAll'
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
                by_score = (va == 0 and vb == 0) or random.random() < self.PF
                if (a.predict < b.predict) if by_score else (va > vb):
                    order[j], order[j + 1] = b, a
                    swapped = True
            if not swapped:
                break
        return order

    def _score(self, children):
        for child, p in zip(children, self.predict(children) if children else []):
            child.predict = p
        return children


class SDGATuner(GATuner):
    """GA whose genotype is decoded into a feasible phenotype by repairing it with the solver
    (SAT-decoding, ga_tuner.py:157-166)."""
    KIND = 'SATDecoding'

    def _score(self, children):
        for child, p in zip(children, self.predict(children) if children else []):
            child.predict = p
        return children
