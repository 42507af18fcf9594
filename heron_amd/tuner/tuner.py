"""Search loop (the role of tuner/tuner.py:47-87 of the reference) and the sampling helpers around it.

A run is a sequence of rounds.  A round refreshes the population (constrained-random samples + best measured points +
the previous population, ranked by predicted score), lets the subclass ``optimize`` it, picks the candidates to
measure, measures them, retrains the cost model and appends a line to ``stat.txt``
(round, sampling s, measuring s, training s, elapsed s, best perf).  What differs between the plain run, the run
with a pre-trained model and the refinement rounds at the end of a constrained-GA run is only how the candidates of a
round are picked, so all three go through ``_round``.
"""
import json
import os
import random
import time

import numpy as np

from ..model import XGBoostCostModel
from ..multi import Job
from ..sample import Sample
from ..utils import Code


def _reseed():
    """Forked workers inherit the parent's generator state; each draws its own."""
    random.seed(int.from_bytes(os.urandom(8), "little"))
    np.random.seed(int.from_bytes(os.urandom(4), "little"))


class Tuner:
    EPSILON = 0.6           # share of a round's candidates taken greedily by prediction (tuner.py:288-298)

    def __init__(self, config):
        self.config = config
        self.iter_no = 0
        self.cost_model = None
        self.total_sample_time = 0
        self.total_measure_time = 0
        self.feasible = None

    def refinement_share(self):
        """Share of the measuring rounds, at the end of a run, whose candidates are the one-knob neighbours of the best
        measured points (the constrained GA switches it on); the reference has no such phase."""
        return 0.0

    def confirmation_tiles(self):
        """Number of distinct block tiles whose best measured points are re-timed, with long repeats, when the search
        is over (0 = no such phase: the reference has none, and only the constrained GA switches it on)."""
        return 0

    # ------------------------------------------------------------------------------------------------ cost model
    def buildCostModel(self, task):
        self.cost_model = XGBoostCostModel(task, self.config)

    def setPretrainedModel(self, model):
        self.cost_model = model

    def predict(self, samples):
        if self.cost_model is None:
            return np.ones(len(samples))
        res = self.cost_model.predict(samples)
        return next(iter(res.values())) if isinstance(res, dict) else res

    def _assign_predictions(self, samples):
        for sample, p in zip(samples, self.predict(samples) if samples else []):
            sample.predict = p
        return samples

    # ------------------------------------------------------------------------------------------------ the rounds
    def _log_round(self, iter_no, t_sample, t_measure, t_train, start_time, env):
        with open(os.path.join(self.config.log_dir, 'stat.txt'), 'a') as f:
            f.write("%d,%f,%f,%f,%f,%f\n" % (iter_no, t_sample, t_measure, t_train, time.time() - start_time,
                                             env.perf_buffer.best_perf or 0))

    def _round(self, env, iter_no, population, stat, start_time, pick, measure=True, train=True, pretrained=False):
        """One round; ``pick(feasible candidates)`` returns the samples to measure.  Returns the new population."""
        print("== Current Round ", iter_no)
        t0 = time.time()
        population, all_pop = self.optimize(env, self.UpdatePopulation(env, population, pretrained), stat, start_time)
        t1 = time.time()
        # points known to violate the constraint system are not worth a build (the reference selects among them
        # too and lets the build fail, tuner.py:66-70)
        chosen = self.FilterSamples(pick([x for x in all_pop if x.valid]), env) if measure else []
        if chosen:
            self.measure(chosen, env)
        t2 = time.time()
        if train and measure and self.cost_model is not None and len(env.perf_buffer.data_y) > 0:
            self.cost_model.train(env.perf_buffer)
        self._log_round(iter_no, t1 - t0, t2 - t1, time.time() - t2, start_time, env)
        return population

    def run_with_pretrained(self, env):
        """Search steered by a model that was fitted beforehand and is not re-trained (tuner.py:32-45):
        ``search_generations`` rounds, each measuring the best-predicted max_trials/generations candidates."""
        self.check_feasible_exits(env)
        start_time = time.time()
        gens = max(1, int(self.config.search_generations))
        per_gen = -(-self.config.max_trials // gens)
        population, stat = [], []
        print("= ---- Tuning with a pre-trained model : Trials %d, Rounds %d ---- =" % (self.config.max_trials, gens))
        for iter_no in range(gens):
            population = self._round(env, iter_no, population, stat, start_time,
                                     lambda cands: self.greedy_select(env, cands, per_gen), train=False, pretrained=True)
        return population, stat

    def run(self, env, do_measure=True):
        self.check_feasible_exits(env)
        start_time = time.time()
        per_round = self.config.measure_time_per_round
        full, rest = divmod(self.config.max_trials, per_round)
        # full rounds, then the remainder (possibly empty, as in tuner.py:50-58); unlike the reference's loop, which
        # adds a round of its own in front of the remainder, a run measures max_trials points, not up to a round more
        quotas = [per_round] * full + [rest]
        measuring = full + (1 if rest else 0)
        refine_from = measuring - (int(self.refinement_share() * measuring + 0.5) if measuring >= 3 else 0)
        population, stat = [], []
        print("= ---- Tuning : Trials %d, Rounds %d ---- =" % (self.config.max_trials, len(quotas)))
        for iter_no, quota in enumerate(quotas):
            if do_measure and quota > 0 and iter_no >= refine_from:
                pick = lambda cands, q=quota: self.refinement_select(env, cands, q)         # noqa: E731
            else:
                pick = lambda cands, q=quota: self.epsilon_select(env, cands, self.EPSILON, q)   # noqa: E731
            population = self._round(env, iter_no, population, stat, start_time, pick, measure=do_measure,
                                     train=iter_no != len(quotas) - 1)
        if do_measure and self.confirmation_tiles() > 0:
            self.confirm(env, self.confirmation_tiles())
        return population, stat

    # ------------------------------------------------------------------------------------------------ confirmation
    def confirmation_candidates(self, env, tiles):
        """The best measured point of each of the ``tiles`` best distinct block tiles, plus - for each - the same tile
        with the wave grid transposed, with the other issue order, and with both: the moves that change a good tile
        by a few percent, which is what separates one search from the next - and the best-predicted variant of each of
        the operator's coupled moves.  The best rows of the records files named
        in ``config.incumbents`` (three confirmed, three others per file) join them."""
        buf = env.perf_buffer
        order = sorted(range(len(buf.data_y)), key=lambda i: -buf.data_y[i])
        bases, seen_tiles = [], set()
        for i in order:
            sample = buf.samples[i]
            pheno = sample.knob_manager.solved_knob_vals_phenotype
            tile = tuple(v for k, v in sorted(pheno.items()) if k.startswith("V#") and k.endswith(("block_m", "block_n")))
            tile += tuple(v for k, v in sorted(pheno.items()) if k.startswith("P#") and k.endswith("block_k_bytes"))
            if tile not in seen_tiles:
                seen_tiles.add(tile)
                bases.append(sample)
            if len(bases) >= tiles:
                break
        out, seen = [], set()

        def consider(knobs):
            s = Sample(env.task)
            point, valid = s.knob_manager.validate(knobs)
            code = Code(point) if valid else None
            if valid and code not in seen:
                seen.add(code)
                s.point, s.valid, s.stmt_code, s.violation = point, True, code, 0
                out.append(s)

        # incumbents of earlier searches (config.incumbents: records files) are re-timed under the same conditions,
        # so a run can only ship something worse than an earlier one if it measures worse today
        probe = Sample(env.task).knob_manager
        for path in getattr(self.config, 'incumbents', None) or []:
            try:
                rows = [json.loads(line) for line in open(path) if line.strip()]
            except OSError:
                print("no incumbents at %s" % path)
                continue
            good = sorted((r for r in rows if r.get("perf", 0) > 0), key=lambda r: -r["perf"])
            for row in [r for r in good if r.get("confirmed")][:3] + [r for r in good if not r.get("confirmed")][:3]:
                consider({n: row["param"].get(n, probe.solver.vals[n].defv) for n in probe.knob_names})

        for base in bases:
            geno = base.knob_manager.solved_knob_vals_genotype
            names = base.knob_manager.knob_names
            twin = {n: n[:-2] + ("_n" if n.endswith("_m") else "_m") for n in names if n.endswith(("_m", "_n"))}
            twin = {n: t for n, t in twin.items() if t in geno and not n.endswith("group_m")}
            order_knob = [n for n in names if n.endswith("issue_order")]
            for transposed in (False, True):
                knobs = {n: geno[twin.get(n, n)] for n in names} if (transposed and twin) else dict(geno)
                consider(dict(knobs))
                for n in order_knob:
                    for cand in base.knob_manager.get_knob_candidates(n):
                        if cand != knobs[n]:
                            consider(dict(knobs, **{n: cand}))
            # the operator's coupled moves (other MFMA edge, other LDS row length at the same block tile): of each kind
            # the feasible variant the cost model likes best, so that a population that settled on the wrong side of a
            # coarse choice still has the other side timed
            moves = getattr(env.task, 'coupled_moves', None)
            groups = {}
            for label, knobs in (moves(base.knob_manager) if moves else []):
                s = Sample(env.task)
                point, valid = s.knob_manager.validate(knobs)
                if valid:
                    s.point, s.valid, s.stmt_code, s.violation = point, True, Code(point), 0
                    groups.setdefault(label, []).append((s, knobs))
            for label, members in groups.items():
                self._assign_predictions([m[0] for m in members])
                consider(max(members, key=lambda m: m[0].predict)[1])
        return out

    def _time_long(self, env, cands, min_repeat_ms, repeat):
        """Times ``cands`` with repeats of at least ``min_repeat_ms`` and files the valid ones as confirmed records."""
        from ..runner.measure import MeasureInput
        from ..runner.runner import perf_of
        runner = env.runner.measure_option.get('runner') if isinstance(env.runner.measure_option, dict) else None
        saved = {}
        for attr, value in (("min_repeat_ms", min_repeat_ms), ("repeat", repeat), ("number", 1)):
            if runner is not None and hasattr(runner, attr):
                saved[attr] = getattr(runner, attr)
                setattr(runner, attr, value)
        try:
            task = env.task
            results = env.runner.measure_batch([MeasureInput(task.target, task, s.knob_manager) for s in cands])
        finally:
            for attr, value in saved.items():
                setattr(runner, attr, value)
        for sample, result in zip(cands, results):
            sample.valid, sample.perf = perf_of(result)
            if sample.valid:
                env.perf_buffer.record_confirmed(sample)
        return [s for s in cands if s.valid]

    def one_knob_neighbours(self, env, base, skip=()):
        """Feasible points that differ from ``base`` in exactly one knob, codes in ``skip`` left out."""
        out, seen = [], set(skip)
        geno = base.knob_manager.solved_knob_vals_genotype
        names = base.knob_manager.knob_names
        for name in names:
            for cand in base.knob_manager.get_knob_candidates(name):
                if cand == geno[name]:
                    continue
                s = Sample(env.task)
                point, valid = s.knob_manager.validate({n: (cand if n == name else geno[n]) for n in names})
                code = Code(point) if valid else None
                if valid and code not in seen:
                    seen.add(code)
                    s.point, s.valid, s.stmt_code, s.violation = point, True, code, 0
                    out.append(s)
        return out

    def confirm(self, env, tiles, min_repeat_ms=100.0, repeat=3):
        """Deterministic end of a search: every confirmation candidate is timed again with repeats of at least
        ``min_repeat_ms`` and filed as a confirmed record; ``Task.apply_best`` prefers confirmed records, so the
        instance a run ships no longer depends on which point a short measurement happened to favour.  Then the best
        confirmed point is polished: all its one-knob neighbours are timed the same way, ``config.polish_rounds`` times
        at most (default 1) and only while the best point keeps moving - the fine knobs (issue order, load spread,
        epilogue, raster group) move a tile by less than a short measurement resolves."""
        cands = self.confirmation_candidates(env, tiles)
        if not cands:
            return []
        print("= ---- Confirmation : %d candidates, repeats of >= %.0f ms ---- =" % (len(cands), min_repeat_ms))
        done = sorted(self._time_long(env, cands, min_repeat_ms, repeat), key=lambda s: -s.perf)
        timed = {s.stmt_code for s in cands}
        for _ in range(int(getattr(self.config, 'polish_rounds', 1))):
            if not done:
                break
            best = done[0]
            near = self.one_knob_neighbours(env, best, skip=timed)
            if not near:
                break
            print("= ---- Polish : %d one-knob neighbours of the confirmed best ---- =" % len(near))
            timed.update(s.stmt_code for s in near)
            done = sorted(done + self._time_long(env, near, min_repeat_ms, repeat), key=lambda s: -s.perf)
            if done[0] is best:
                break
        if done:
            print("confirmed best %f (latency %.6f ms)" % (done[0].perf, 1e3 * np.exp(-done[0].perf)))
        return done

    def optimize(self, env, population, stat, s_time):
        raise NotImplementedError()

    def measure(self, samples, env):
        env.evalSamples(samples)

    # ------------------------------------------------------------------------------------------------ population
    def UpdatePopulation(self, env, population, pretrained=False):
        fresh = self.constrained_random_sample(env, self.config.pop_num)
        veterans = self.history_topk_samples(env, self.config.history_topk)
        if not pretrained:
            self.repredict(population)      # the cost model has changed since these were scored
        ranked = sorted(population + veterans + fresh, key=lambda x: -x.predict)[: self.config.pop_num]
        scores = np.array([x.predict for x in ranked])
        print('PMAX %f, PMin %f, NUM %d' % (scores.max(), scores.min(), len(scores)))
        return ranked

    def history_topk_samples(self, env, k):
        """The k best measured samples, worst of them first."""
        buf = env.perf_buffer
        order = sorted(range(len(buf.data_y)), key=lambda i: buf.data_y[i])[-k:] if k > 0 else []
        best = [buf.samples[i] for i in order]
        for sample in best:
            sample.violation = 0.0
        return best

    def repredict(self, pop):
        for sample in pop:
            sample.predict = self.predict([sample])[0] if sample.valid else 0.0
            if sample.valid:
                sample.violation = 0.0

    def incumbent_neighbours(self, env, top=3):
        """Feasible points that differ from one of the ``top`` best measured points in exactly one knob (the solver
        re-derives the dependent variables), scored by the cost model."""
        out, seen = [], set()

        def consider(knobs):
            s = Sample(env.task)
            point, valid = s.knob_manager.validate(knobs)
            code = Code(point) if valid else None
            if valid and code not in seen:
                seen.add(code)
                s.point, s.valid, s.stmt_code, s.violation = point, True, code, 0
                out.append(s)

        for base in reversed(self.history_topk_samples(env, top)):
            geno = base.knob_manager.solved_knob_vals_genotype
            names = base.knob_manager.knob_names
            for name in names:
                for cand in base.knob_manager.get_knob_candidates(name):
                    if cand != geno[name]:
                        consider({n: (cand if n == name else geno[n]) for n in names})
            # one coupled move that no single knob reaches: the same block tile with the wave grid transposed
            # (knobs named ..._m / ..._n in pairs swap their values)
            twin = {n: n[:-2] + ("_n" if n.endswith("_m") else "_m") for n in names if n.endswith(("_m", "_n"))}
            twin = {n: t for n, t in twin.items() if t in geno and not n.endswith("group_m")}
            if twin:
                consider({n: geno[twin.get(n, n)] for n in names})
            # and the operator's own coupled moves (other MFMA edge at the same block tile, other LDS row length with
            # every stage count): the coarse choices a population can settle on the wrong side of
            moves = getattr(env.task, 'coupled_moves', None)
            for _, knobs in (moves(base.knob_manager) if moves else []):
                consider(knobs)
        return self._assign_predictions(out)

    # ------------------------------------------------------------------------------------------------ feasibility table
    def check_feasible_exits(self, env, sample_num=1e3):
        """Per-knob feasible value sets for the unconstrained operators, cached in feasible.json
        (tuner.py:115-144); the constrained tuners override this with a no-op."""
        path = self.config.feasible_file_path
        wanted = set(env.task.knob_manager.solver.vals.keys())
        if os.path.exists(path):
            with open(path) as f:
                cached = json.load(f)
            # a file left by another task or an older constraint set does not cover this task's variables
            if set(cached) == wanted:
                self.feasible = cached
                return
        print("Feasible not exists, random sample for the first time.")
        count = int(getattr(self.config, 'feasible_samples', sample_num))
        seen = {}
        for sample in self.constrained_random_sample(env, count, timeout=200):
            for name, value in sample.knob_manager.solved_knob_vals_phenotype.items():
                seen.setdefault(name, set()).add(value)
        self.feasible = {name: sorted(values) for name, values in seen.items()}
        with open(path, 'w') as f:
            json.dump(self.feasible, f)

    # ------------------------------------------------------------------------------------------------ selection
    def RouletteWheelSelection(self, samples, num):
        """``num`` draws with replacement, probability proportional to the score above the worst."""
        if len(samples) <= num:
            return samples
        w = np.array([x.predict for x in samples], dtype=np.float64)
        w = w - w.min() + 1e-16
        return [samples[i] for i in np.random.choice(len(samples), num, p=w / w.sum(), replace=True)]

    def RankSelection(self, samples, num):
        """``num`` distinct draws, probability falling linearly with the position in ``samples``."""
        if len(samples) <= num:
            return samples
        w = np.arange(len(samples), 0, -1, dtype=np.float64)
        return [samples[i] for i in np.random.choice(len(samples), num, p=w / w.sum(), replace=False)]

    def recordStat(self, samples, env, start_time, stat):
        fresh = self.FilterSamples(samples, env)
        if not fresh:
            return
        scores = sorted((x.predict for x in fresh), reverse=True)
        top5 = scores[:5]
        elapsed = time.time() - start_time
        stat.append([elapsed, scores[0], sum(top5) / len(top5)])
        print("Time %f, MAX %f, TOP5_MEAN %f" % (elapsed, scores[0], sum(top5) / len(top5)))

    def FilterSamples(self, samples, env):
        """Drops duplicates and points that were measured before (same order otherwise)."""
        taken, kept = set(env.perf_buffer.perfs), []
        for sample in samples:
            if sample.stmt_code not in taken:
                taken.add(sample.stmt_code)
                kept.append(sample)
        return kept

    def _ranked_unmeasured(self, env, samples):
        ranked = sorted(self.FilterSamples(samples, env), key=lambda x: -x.predict)
        if ranked:
            print("Best predicted ", ranked[0].predict)
        return ranked

    def greedy_select(self, env, all_samples, select_num):
        return self._ranked_unmeasured(env, all_samples)[:select_num]

    def epsilon_select(self, env, all_samples, epsilon, select_num):
        """Top ``epsilon`` share by prediction, the rest by roulette wheel (tuner.py:288-298)."""
        ranked = self._ranked_unmeasured(env, all_samples)
        k = int(select_num * epsilon)
        return ranked[:k] + (self.RouletteWheelSelection(ranked[k:], select_num - k) if ranked else [])

    def refinement_select(self, env, all_samples, select_num):
        """The best-predicted unmeasured one-knob neighbours of the incumbents; the GA's candidates fill what is left."""
        near = self.greedy_select(env, self.incumbent_neighbours(env), select_num)
        print("refinement round: %d unmeasured one-knob neighbours of the best points" % len(near))
        if len(near) >= select_num:
            return near
        mine = {n.stmt_code for n in near}
        rest = [x for x in all_samples if x.stmt_code not in mine]
        return near + self.epsilon_select(env, rest, self.EPSILON, select_num - len(near))

    # ------------------------------------------------------------------------------------------------ sampling
    def constrained_random_sample(self, env, number, timeout=10):
        if self.config.parallel:
            samples = constrained_random_sample_parallel(env.task, number, self.config, timeout)
            if not samples:
                # every sampler child failed or timed out: do a smaller batch in this process so the search goes on
                print("warning: parallel sampling returned nothing, sampling %d points in-process" % min(number, 32))
                samples = constrained_random_sample_sequential(env.task, min(number, 32), self.config)
        else:
            samples = constrained_random_sample_sequential(env.task, number, self.config)
        for sample in self._assign_predictions(samples):
            sample.violation = 0
        return samples

    def constrained_random_walk(self, task, pop, num_per_sample, ratio=0.3):
        walk = random_walk_parallel if self.config.parallel else random_walk_sequential
        return self._assign_predictions(walk('constrained_random_walk', task, pop, num_per_sample, [ratio]))


# ---------------------------------------------------------------------------------------------------- worker jobs
def _run_jobs(jobs):
    """Starts every job, then collects what they return (a job that died or timed out contributes nothing)."""
    for job in jobs:
        job.start(job.attach_info)
    gathered = []
    for job in jobs:
        part = job.get()
        if isinstance(part, list):
            gathered.extend(part)
    return gathered


def _finish(sample, point, valid):
    sample.point, sample.valid, sample.stmt_code = point, bool(valid), Code(point)
    return sample


def constrained_random_sample_sequential(task, number, config):
    _reseed()
    out = []
    for _ in range(number):
        sample = Sample(task)
        try:
            valid, point = sample.knob_manager.randSample({})
        except RuntimeError:
            continue                # the search gave up on this draw; the rest of the batch is still worth having
        out.append(_finish(sample, point, valid))
    return out


def constrained_random_sample_parallel(task, number, config, timeout):
    share = -(-number // config.parallel_num)
    return _run_jobs([Job(constrained_random_sample_sequential, (task, share, config), timeout)
                      for _ in range(config.parallel_num)])


def random_walk_sequential(kind, task, pop, num_per_sample, args):
    """``num_per_sample`` neighbours of every member of ``pop``: 'random_walk' changes one knob to a value of the
    feasible-value table and validates, 'constrained_random_walk' keeps a share of the variables and re-solves."""
    if kind not in ('random_walk', 'constrained_random_walk'):
        raise ValueError(kind)
    _reseed()
    out = []
    for parent in pop:
        for _ in range(num_per_sample):
            sample = Sample(task)
            point, valid = getattr(sample.knob_manager, kind)(parent.knob_manager, *args)
            out.append(_finish(sample, point, valid))
    return out


def random_walk_parallel(kind, task, pop, num_per_sample, args, timeout=100, parallel_num=4):
    share = -(-len(pop) // parallel_num) if pop else 0
    chunks = [pop[i * share:(i + 1) * share] for i in range(parallel_num)]
    return _run_jobs([Job(random_walk_sequential, (kind, task, chunk, num_per_sample, args), timeout)
                      for chunk in chunks])
