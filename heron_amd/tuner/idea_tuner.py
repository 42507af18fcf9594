"""Infeasibility-driven evolutionary tuner (tuner/idea_tuner.py:11-157 of the reference).

Children come from simulated-binary crossover over all CSP variables and may be infeasible.  Feasible and
infeasible individuals are ranked separately by non-dominated sorting on two objectives (predicted score, and a
constraint-violation measure: the sum over constraints of the individual's rank in that constraint's violation),
ties inside a front broken by crowding distance; the next population keeps a share ``alpha`` of infeasible
individuals close to the constraint boundary.  Infeasible samples are never measured (their score is zeroed
before selection).
"""
import time

import numpy as np

from .ga_tuner import _offspring
from .tuner import Tuner


class IDEATuner(Tuner):
    ALPHA = 0.2

    def optimize(self, env, pop, stat, s_time):
        n_inf = int(self.ALPHA * len(pop))
        n_f = len(pop) - n_inf
        all_pop = [] + pop
        for _ in range(self.config.iter_walks):
            if hasattr(self.cost_model, 'bst') and self.cost_model.bst is None:
                break
            t0 = time.time()
            children = self.crossoverAndMutate(pop, env.task)
            feasible = [p for p in pop + children if p.valid]
            infeasible = [p for p in pop + children if not p.valid]
            pop = self.Rank(feasible)[:n_f] + self.Rank(infeasible)[:n_inf]
            all_pop += children
            stat.append([float(np.max([x.predict for x in all_pop])), time.time() - s_time])
            print(" IDEA iteration time ", time.time() - t0)
        for sample in all_pop:
            if not sample.valid:
                sample.predict = 0.0
        return pop, all_pop

    def UpdatePopulation(self, env, population, pretrained=False):
        """Half of the population from (previous + best measured), half from fresh constrained-random samples."""
        topk = self.history_topk_samples(env, self.config.history_topk)
        rand = self.constrained_random_sample(env, self.config.pop_num)
        if not pretrained:
            self.repredict(population)
        half = self.config.pop_num // 2
        pop = sorted(population + topk, key=lambda x: -x.predict)[:half] + sorted(rand, key=lambda x: -x.predict)[:half]
        perfs = np.array([x.predict for x in pop])
        print('PMAX %f, PMin %f, NUM %d' % (perfs.max(), perfs.min(), len(perfs)))
        return pop

    # --- ranking -------------------------------------------------------------------------------------
    @staticmethod
    def constraint_measure(pop):
        dim = len(pop[0].knob_manager.solver.primitives)
        for p in pop:
            v = getattr(p, 'violations', None)
            if v is None:
                v = [0] * dim if p.valid else [1e8] * dim
            p.violations = list(v)
        ranks = np.zeros((len(pop), dim))
        for i in range(dim):
            col = np.array([p.violations[i] for p in pop], dtype=np.float64)
            _, dense = np.unique(col, return_inverse=True)          # equal violations share a rank
            ranks[:, i] = dense
        for p, r in zip(pop, ranks.sum(axis=1)):
            p.rank = float(r)

    def Rank(self, pop):
        """Non-dominated sorting on (predict high, constraint measure) followed by crowding distance."""
        if not pop:
            return []
        self.constraint_measure(pop)
        n = len(pop)
        f = np.array([[p.predict, p.rank] for p in pop], dtype=np.float64)
        dominated_by = [[] for _ in range(n)]
        count = np.zeros(n, dtype=int)
        for i in range(n):
            for j in range(i + 1, n):
                ge, le = np.all(f[i] >= f[j]), np.all(f[j] >= f[i])
                if ge and not le:
                    dominated_by[i].append(j); count[j] += 1
                elif le and not ge:
                    dominated_by[j].append(i); count[i] += 1
        front = [i for i in range(n) if count[i] == 0]
        ordered = []
        while front:
            self.crowding(pop, front, f)
            ordered += sorted(front, key=lambda i: pop[i].dist)
            nxt = []
            for i in front:
                for j in dominated_by[i]:
                    count[j] -= 1
                    if count[j] == 0:
                        nxt.append(j)
            front = nxt
        return [pop[i] for i in ordered]

    @staticmethod
    def crowding(pop, front, f):
        for i in front:
            pop[i].dist = 0.0
        for obj in range(f.shape[1]):
            order = sorted(front, key=lambda i: f[i, obj])
            span = f[order[-1], obj] - f[order[0], obj] + 1e-8
            if obj == 0:
                pop[order[0]].dist = pop[order[-1]].dist = 1e8
            for k in range(1, len(order) - 1):
                pop[order[k]].dist += (f[order[k + 1], obj] - f[order[k - 1], obj]) / span

    def crossoverAndMutate(self, samples, task):
        res = _offspring(self.config, 'SBX', samples, task, self.feasible)
        valid = [s for s in res if s.valid]
        if valid:
            for s, p in zip(valid, self.predict(valid)):
                s.predict = p
        for s in res:
            if not s.valid:
                s.predict = 0
        return res
