"""Search loop (tuner/tuner.py:47-87 of the reference) and the sampling helpers around it.

Per round: refresh the population (constrained-random samples + best measured + previous
population, ranked by predicted score), ``optimize`` it (subclass), pick ``measure_time_per_round``
candidates with epsilon-greedy selection, measure, retrain the cost model, append a line to
``stat.txt`` (iter, sample_s, measure_s, train_s, elapsed_s, best_perf).
"""
import json
import math
import os
import time

import numpy as np

from ..model import XGBoostCostModel
from ..multi import Job
from ..sample import Sample
from ..utils import Code


class Tuner:
    def __init__(self, config):
        self.config = config
        self.iter_no = 0
        self.cost_model = None
        self.total_sample_time = 0
        self.total_measure_time = 0
        self.feasible = None
        # share of the measuring rounds, at the end of a run, whose candidates are the one-knob neighbours of the best
        # measured points (constrained tuners switch it on); the reference has no such phase
        self.refine_share = 0.0

    def buildCostModel(self, task):
        self.cost_model = XGBoostCostModel(task, self.config)

    def setPretrainedModel(self, model):
        self.cost_model = model

    def predict(self, samples):
        if self.cost_model is None:
            return np.ones(len(samples))
        res = self.cost_model.predict(samples)
        if isinstance(res, dict):
            return res[list(res.keys())[0]]
        return res

    def run_with_pretrained(self, env):
        """Search steered by a model that was fitted beforehand and is not re-trained (tuner.py:32-45):
        ``search_generations`` rounds, each measuring the best-predicted max_trials/generations candidates."""
        self.check_feasible_exits(env)
        start_time = time.time()
        gens = max(1, int(self.config.search_generations))
        population, stat = [], []
        print("= ---- Tuning with a pre-trained model : Trials %d, Rounds %d ---- =" % (self.config.max_trials, gens))
        for iter_no in range(gens):
            print("== Current Round ", iter_no)
            sample_s = time.time()
            initial_population = self.UpdatePopulation(env, population, True)
            population, all_pop = self.optimize(env, initial_population, stat, start_time)
            sample_e = time.time()
            pop = self.greedy_select(env, [x for x in all_pop if x.valid], math.ceil(self.config.max_trials / gens))
            if pop:
                self.measure(pop, env)
            with open(os.path.join(self.config.log_dir, 'stat.txt'), 'a') as f:
                best_perf = env.perf_buffer.best_perf or 0
                f.write("%d,%f,%f,%f,%f,%f\n" % (iter_no, sample_e - sample_s, time.time() - sample_e, 0.0,
                                                 time.time() - start_time, best_perf))
        return population, stat

    def run(self, env, do_measure=True):
        self.check_feasible_exits(env)
        start_time = time.time()
        per_round = self.config.measure_time_per_round
        total_iters = math.ceil(self.config.max_trials / per_round) + 1
        last_iter_select_num = self.config.max_trials % per_round
        population = []
        stat = []
        print("= ---- Tuning : Trials %d, Rounds %d ---- =" % (self.config.max_trials, total_iters))
        for iter_no in range(total_iters):
            select_num = last_iter_select_num if iter_no == total_iters - 1 else per_round
            print("== Current Round ", iter_no)
            sample_s = time.time()
            initial_population = self.UpdatePopulation(env, population)
            population, all_pop = self.optimize(env, initial_population, stat, start_time)
            sample_e = time.time()

            measure_s = time.time()
            # points known to violate the constraint system are not worth a build (the reference selects among them
            # too and lets the build fail, tuner.py:66-70)
            measuring_rounds = total_iters - (1 if last_iter_select_num == 0 else 0)
            refine_rounds = int(self.refine_share * measuring_rounds + 0.5) if measuring_rounds >= 3 else 0
            if do_measure and select_num > 0 and iter_no >= measuring_rounds - refine_rounds:
                near = self.greedy_select(env, self.incumbent_neighbours(env), select_num)
                print("refinement round: %d unmeasured one-knob neighbours of the best points" % len(near))
                rest = [x for x in all_pop if x.valid and x.stmt_code not in {n.stmt_code for n in near}]
                pop = near + self.epsilon_select(env, rest, 0.6, select_num - len(near)) if len(near) < select_num else near
            else:
                pop = self.epsilon_select(env, [x for x in all_pop if x.valid], 0.6, select_num)
            if do_measure and pop != []:
                samples = self.FilterSamples(pop, env)
                self.measure(samples, env)
            measure_e = time.time()

            train_s = time.time()
            if iter_no != total_iters - 1 and self.cost_model is not None and len(env.perf_buffer.data_y) > 0 \
                    and do_measure:
                self.cost_model.train(env.perf_buffer)
            train_e = time.time()
            with open(os.path.join(self.config.log_dir, 'stat.txt'), 'a') as f:
                best_perf = env.perf_buffer.best_perf
                if best_perf is None:
                    best_perf = 0
                f.write("%d,%f,%f,%f,%f,%f\n" % (iter_no, sample_e - sample_s, measure_e - measure_s,
                                                 train_e - train_s, time.time() - start_time, best_perf))
        return population, stat

    def optimize(self, env, population, stat, s_time):
        raise NotImplementedError()

    def UpdatePopulation(self, env, population, pretrained=False):
        rand = self.constrained_random_sample(env, self.config.pop_num)
        topk = self.history_topk_samples(env, self.config.history_topk)
        if not pretrained:
            self.repredict(population)      # the cost model has changed since these were scored
        all_pop = population + topk + rand
        pop_sorted = sorted(all_pop, key=lambda x: -x.predict)
        ret = pop_sorted[: self.config.pop_num]
        perfs = np.array([x.predict for x in ret])
        print('PMAX %f, PMin %f, NUM %d' % (perfs.max(), perfs.min(), len(perfs)))
        return ret

    def measure(self, samples, env):
        env.evalSamples(samples)

    def check_feasible_exits(self, env, sample_num=1e3):
        """Per-knob feasible value sets for the unconstrained operators, cached in feasible.json
        (tuner.py:115-144); the constrained tuners override this with a no-op."""
        path = self.config.feasible_file_path
        if os.path.exists(path):
            with open(path, 'r') as f:
                cached = json.loads(f.read())
            # a file left by another task or an older constraint set does not cover this task's variables
            if set(cached.keys()) == set(env.task.knob_manager.solver.vals.keys()):
                self.feasible = cached
                return
        print("Feasible not exists, random sample for the first time.")
        sample_num = getattr(self.config, 'feasible_samples', sample_num)
        population = self.constrained_random_sample(env, int(sample_num), timeout=200)
        dict_set = {}
        for sample in population:
            for valname, val in sample.knob_manager.solved_knob_vals_phenotype.items():
                dict_set.setdefault(valname, set()).add(val)
        dict_list = {key: sorted(vals) for key, vals in dict_set.items()}
        with open(path, 'w') as f:
            f.write(json.dumps(dict_list))
        self.feasible = dict_list

    def RouletteWheelSelection(self, samples, num):
        if len(samples) <= num:
            return samples
        predicts = np.array([x.predict for x in samples], dtype=np.float64)
        predicts_ = predicts - predicts.min() + 1e-16
        probs = predicts_ / predicts_.sum()
        idx = np.random.choice(len(samples), num, p=probs, replace=True)
        return [samples[i] for i in idx]

    def RankSelection(self, samples, num):
        if len(samples) <= num:
            return samples
        predicts_ = (len(samples) - np.arange(len(samples))).astype(np.float64)
        probs = predicts_ / predicts_.sum()
        idx = np.random.choice(len(samples), num, p=probs, replace=False)
        return [samples[i] for i in idx]

    def recordStat(self, samples, env, start_time, stat):
        samples = self.FilterSamples(samples, env)
        if not samples:
            return
        perfs = sorted([x.predict for x in samples], key=lambda x: -x)
        max_perf = perfs[0]
        top5_mean = sum(perfs[:5]) / len(perfs[:5])
        time_point = time.time() - start_time
        stat.append([time_point, max_perf, top5_mean])
        print("Time %f, MAX %f, TOP5_MEAN %f" % (time_point, max_perf, top5_mean))

    def FilterSamples(self, samples, env):
        codes = set()
        ret = []
        for sample in samples:
            code = sample.stmt_code
            if code in codes or code in env.perf_buffer.perfs:
                continue
            codes.add(code)
            ret.append(sample)
        return ret

    def constrained_random_sample(self, env, number, timeout=10):
        if self.config.parallel:
            samples = constrained_random_sample_parallel(env.task, number, self.config, timeout)
            if not samples:
                # every sampler child failed or timed out: do a smaller batch in this process so the search goes on
                print("warning: parallel sampling returned nothing, sampling %d points in-process" % min(number, 32))
                samples = constrained_random_sample_sequential(env.task, min(number, 32), self.config)
        else:
            samples = constrained_random_sample_sequential(env.task, number, self.config)
        perfs = self.predict(samples)
        for idx, sample in enumerate(samples):
            sample.predict = perfs[idx]
            sample.violation = 0
        return samples

    def constrained_random_walk(self, task, pop, num_per_sample, ratio=0.3):
        if self.config.parallel:
            samples = random_walk_parallel('constrained_random_walk', task, pop, num_per_sample, [ratio, ])
        else:
            samples = random_walk_sequential('constrained_random_walk', task, pop, num_per_sample, [ratio, ])
        perfs = self.predict(samples)
        for idx, sample in enumerate(samples):
            sample.predict = perfs[idx]
        return samples

    def history_topk_samples(self, env, k):
        p = list(zip(env.perf_buffer.data_x, env.perf_buffer.data_y, env.perf_buffer.samples))
        ps = sorted(p, key=lambda x: x[1])[-k:]
        ret = []
        for _, _, sample in ps:
            sample.violation = 0.0
            ret.append(sample)
        return ret

    def incumbent_neighbours(self, env, top=3):
        """Feasible points that differ from one of the ``top`` best measured points in exactly one knob (the solver
        re-derives the dependent variables), scored by the cost model."""
        out, seen = [], set()
        for base in reversed(self.history_topk_samples(env, top)):
            geno = base.knob_manager.solved_knob_vals_genotype
            names = base.knob_manager.knob_names
            for name in names:
                for cand in base.knob_manager.get_knob_candidates(name):
                    if cand == geno[name]:
                        continue
                    s = Sample(env.task)
                    point, valid = s.knob_manager.validate({n: (cand if n == name else geno[n]) for n in names})
                    if not valid:
                        continue
                    s.point, s.valid, s.stmt_code = point, True, Code(point)
                    if s.stmt_code in seen:
                        continue
                    seen.add(s.stmt_code)
                    out.append(s)
        perfs = self.predict(out) if out else []
        for s, p in zip(out, perfs):
            s.predict, s.violation = p, 0
        return out

    def repredict(self, pop):
        for sample in pop:
            if sample.valid:
                sample.predict = self.predict([sample])[0]
                sample.violation = 0.0
            else:
                sample.predict = 0.0

    def greedy_select(self, env, all_samples, select_num):
        filtered = self.FilterSamples(all_samples, env)
        if len(filtered) == 0:
            return []
        _sorted = sorted(filtered, key=lambda x: -x.predict)
        print("Best predicted ", _sorted[0].predict)
        return _sorted[:select_num]

    def epsilon_select(self, env, all_samples, epsilon, select_num):
        """Top ``epsilon`` share by prediction, the rest by roulette wheel (tuner.py:288-298)."""
        filtered = self.FilterSamples(all_samples, env)
        if len(filtered) == 0:
            return []
        _sorted = sorted(filtered, key=lambda x: -x.predict)
        print("Best predicted ", _sorted[0].predict)
        k = int(select_num * epsilon)
        topk = _sorted[:k]
        left = _sorted[k:]
        return topk + self.RouletteWheelSelection(left, select_num - k)


def _run_jobs(jobs):
    for job in jobs:
        job.start(job.attach_info)
    res = []
    for job in jobs:
        ret = job.get()
        if isinstance(ret, list):
            res += ret
    return res


def constrained_random_sample_parallel(task, number, config, timeout):
    work_load = int((number + config.parallel_num - 1) // config.parallel_num)
    jobs = [Job(constrained_random_sample_sequential, (task, work_load, config), timeout)
            for _ in range(config.parallel_num)]
    return _run_jobs(jobs)


def constrained_random_sample_sequential(task, number, config):
    import random
    random.seed(int.from_bytes(os.urandom(8), "little"))      # forked workers must not share a stream
    np.random.seed(int.from_bytes(os.urandom(4), "little"))
    ret = []
    for _ in range(number):
        sample = Sample(task)
        valid, point = sample.knob_manager.randSample({})
        sample.point = point
        sample.valid = valid
        sample.stmt_code = Code(point)
        ret.append(sample)
    return ret


def random_walk_parallel(kind, task, pop, num_per_sample, args, timeout=100, parallel_num=4):
    work_load = int((len(pop) + parallel_num - 1) // parallel_num)
    jobs = []
    for i in range(parallel_num):
        chunk = pop[i * work_load: (i + 1) * work_load]
        jobs.append(Job(random_walk_sequential, (kind, task, chunk, num_per_sample, args), timeout))
    return _run_jobs(jobs)


def random_walk_sequential(kind, task, pop, num_per_sample, args):
    import random
    random.seed(int.from_bytes(os.urandom(8), "little"))
    np.random.seed(int.from_bytes(os.urandom(4), "little"))
    ret = []
    for sample in pop:
        for _ in range(num_per_sample):
            new_sample = Sample(task)
            if kind == 'random_walk':
                point, valid = new_sample.knob_manager.random_walk(sample.knob_manager, *args)
            elif kind == 'constrained_random_walk':
                point, valid = new_sample.knob_manager.constrained_random_walk(sample.knob_manager, *args)
            else:
                raise ValueError(kind)
            new_sample.point = point
            new_sample.valid = bool(valid)
            new_sample.stmt_code = Code(point)
            ret.append(new_sample)
    return ret
