"""Knob registry and constraint builders over the CSP solver.

Interface of the reference's KnobManager (schedule/constraints/ortools/knobManager.py:15-484):
variables and knobs are registered while the template is being *built* (``is_building``),
each builder appends primitives to ``solver.primitives``; afterwards ``randSample``,
``validate`` and the crossover / random-walk operators produce assignments
(``solved_knob_vals_genotype`` / ``_phenotype``) that ``get_val`` serves when a template is
instantiated.
"""
import math
import random

import numpy as np

from .primitives import EQ, LE, LT, NE, ProdTwo, Sum
from .solver import Solver


def str_vec(vec):
    return "[" + "".join(str(i) + "," for i in vec) + "]"


class KnobManager:
    def __init__(self):
        self.sched_tups = []
        self.is_building = True
        self.solver = Solver()

        self.axis_parents = {}
        self.axis_brother = {}
        self.axis_ori_lenth = {}
        self.mems = []
        self.staged_fused_axes = set()

        self.knob_names = []
        self.solved_knob_vals_genotype = {}
        self.solved_knob_vals_phenotype = {}
        self.candidates = {}
        self._valid = False

        self.constraint_descs = ""
        self.dump_descs = False

    # ------------------------------------------------------------------ values
    def get_val(self, name):
        if isinstance(name, int):
            return name
        assert isinstance(name, str)
        if name in self.axis_ori_lenth.keys() and name not in self.staged_fused_axes:
            return self.axis_ori_lenth[name]
        if self.is_building:
            return self.solver.vals[name].defv
        return self.solved_knob_vals_phenotype.get(name)

    def define_value(self, name, low, up, def_val, is_knob=False):
        if not self.is_building:
            return name
        if name in self.solver.vals.keys():
            return name
        if is_knob:
            self.knob_names.append(name)
        self.solver.addVal(name, low, up, def_val)
        return name

    def get_ax(self, ax):
        """A variable name, or the constant extent of an un-split axis."""
        if ax in self.solver.vals.keys():
            return ax
        if ax in self.axis_ori_lenth and ax not in self.staged_fused_axes:
            return self.axis_ori_lenth[ax]
        raise KeyError(ax)

    def changeUp(self, a, b):
        self.solver.vals[a].up = min(self.solver.vals[a].up, b)

    def changeLow(self, a, b):
        self.solver.vals[a].low = max(self.solver.vals[a].low, b)

    def _desc(self, s):
        if self.dump_descs:
            self.constraint_descs += s

    # ------------------------------------------------------------------ constraint builders
    def addSplitFactor(self, ax_key, axo_key, axi_key, knob):
        """ax = axo * axi with the inner extent tied to ``knob`` (knobManager.py:83-94)."""
        if not self.is_building:
            return
        self.solver.primitives.append(ProdTwo([self.get_ax(ax_key), [self.get_ax(axo_key), self.get_ax(axi_key)]]))
        self.solver.primitives.append(EQ([self.get_ax(axi_key), knob]))
        self.axis_brother[axi_key] = axo_key
        self.axis_brother[axo_key] = axi_key
        self._desc("&Prod(%s,%s)&EQ(%s,%s)" % (ax_key, str_vec([axo_key, axi_key]), axi_key, knob))

    def addSplitNparts(self, ax_key, axo_key, axi_key, knob):
        if not self.is_building:
            return
        self.solver.primitives.append(ProdTwo([self.get_ax(ax_key), [self.get_ax(axo_key), self.get_ax(axi_key)]]))
        self.solver.primitives.append(EQ([self.get_ax(axo_key), knob]))
        self.axis_brother[axi_key] = axo_key
        self.axis_brother[axo_key] = axi_key
        self._desc("&Prod(%s,%s)&EQ(%s,%s)" % (ax_key, str_vec([axo_key, axi_key]), axo_key, knob))

    def addProd(self, src, res):
        """res == product(src); longer products are chained through temporaries (knobManager.py:114-141)."""
        if not self.is_building:
            return
        if len(src) == 1:
            self.solver.primitives.append(EQ([src[0], res]))
        elif len(src) == 2:
            self.solver.primitives.append(ProdTwo([res, [src[0], src[1]]]))
        else:
            a = src[0]
            up = self.solver.vals[res].up if isinstance(res, str) else res
            for i in range(len(src) - 2):
                temp = str(a) + '_' + str(src[i + 1])
                self.define_value(temp, 0, up, 1)
                self.solver.primitives.append(ProdTwo([temp, [a, src[i + 1]]]))
                a = temp
            self.solver.primitives.append(ProdTwo([res, [a, src[-1]]]))
        self._desc("&Prod(%s,%s)" % (res, str_vec(src)))

    def addLE(self, a, b):
        if not self.is_building:
            return
        assert isinstance(a, str)
        if isinstance(b, str):
            self.solver.primitives.append(LE([a, b]))
        else:
            self.changeUp(a, b)
        self._desc("&LE(%s,%s)" % (a, b))

    def addEQ(self, a, b):
        if not self.is_building:
            return
        assert isinstance(a, str)
        if isinstance(b, str):
            self.solver.primitives.append(EQ([a, b]))
        else:
            self.changeUp(a, b)
            self.changeLow(a, b)
        self._desc("&EQ(%s,%s)" % (a, b))

    def addNE(self, a, b):
        if not self.is_building:
            return
        self.solver.primitives.append(NE([a, b]))
        self._desc("&NE(%s,%s)" % (a, b))

    def addLT(self, a, b):
        if not self.is_building:
            return
        assert isinstance(a, str)
        if isinstance(b, str):
            self.solver.primitives.append(LT([a, b]))
        else:
            self.changeUp(a, b - 1)
        self._desc("&LT(%s,%s)" % (a, b))

    def addSelect(self, cand_keys, knob_key, val_key):
        """val == cand_keys[knob] through one 0/1 selector per candidate (knobManager.py:189-207)."""
        if not self.is_building:
            return
        up = min(len(cand_keys) - 1, self.solver.vals[knob_key].up)
        keys = []
        for i in range(up + 1):
            key = (knob_key + '_select%d' % i)
            assert "P#" in knob_key
            key = key.replace("P#", "O#")
            self.define_value(key, 0, 1, 0)
            self.solver.primitives.append(EQ([val_key, cand_keys[i]], cond=key))
            self.solver.primitives.append(EQ([knob_key, i], cond=key))
            keys.append(key)
        self.solver.primitives.append(Sum([1, keys]))
        self._desc("&SELECT(%s,%s,%s)" % (val_key, knob_key, str_vec(cand_keys)))

    def addSUM(self, resname, keys):
        if not self.is_building:
            return
        self.solver.primitives.append(Sum([resname, keys]))
        self._desc("&SUM(%s,%s)" % (resname, str_vec(keys)))

    def addCandidates(self, valname, candidates):
        """valname takes one of ``candidates`` (one 0/1 indicator each; knobManager.py:217-236)."""
        if not self.is_building:
            return
        idxs = []
        for idx, v in enumerate(candidates):
            idx_name = valname + '_cand%d' % idx
            idx_name = idx_name.replace("P#", "O#") if "P#" in valname else "O#" + idx_name
            self.define_value(idx_name, 0, 1, 0)
            self.solver.primitives.append(EQ([valname, v], cond=idx_name))
            idxs.append(idx_name)
        self.solver.primitives.append(Sum([1, idxs]))
        if valname in self.knob_names:
            self.candidates[valname] = list(candidates)
        self._desc("&IN(%s,%s)" % (valname, str_vec(candidates)))

    def addRawCandidates(self, valname, candidates):
        if not self.is_building:
            return
        self.candidates[valname] = list(candidates)

    def get_knob_candidates(self, name):
        if name in self.candidates.keys():
            return self.candidates[name]
        low, up = self.solver.vals[name].low, self.solver.vals[name].up
        assert up - low + 1 <= 30
        return list(range(low, up + 1))

    # ------------------------------------------------------------------ sampling
    def _store(self, point):
        for idx, key in enumerate(list(self.solver.vals.keys())):
            self.solved_knob_vals_genotype[key] = point[idx]
            self.solved_knob_vals_phenotype[key] = point[idx]

    def randSample(self, known={}, bounds={}):
        """Random hints for every knob, then the first feasible point (knobManager.py:296-310)."""
        hint = {}
        for key in self.knob_names:
            if key in known.keys():
                continue
            candidates = self.get_knob_candidates(key)
            hint[key] = candidates[random.randint(0, len(candidates) - 1)]
        valid, point = self.solver.solve(hint=hint, known=known, bounds=bounds)
        for _ in range(3):
            if valid or self.solver.last_status != 'unknown':
                break
            # the randomised search gave up, which proves nothing: try again from other hints
            hint = {k: random.choice(self.get_knob_candidates(k)) for k in hint}
            valid, point = self.solver.solve(hint=hint, known=known, bounds=bounds)
        if not valid:
            raise RuntimeError("no feasible point (%s)" % self.solver.last_status)
        self._valid = valid
        self._store(point)
        return valid, point

    def validate(self, knob_dict):
        valid, point = self.solver.validate(knob_dict)
        self._valid = valid
        if valid:
            self._store(point)
        else:
            for key in knob_dict.keys():
                self.solved_knob_vals_genotype[key] = knob_dict[key]
                self.solved_knob_vals_phenotype[key] = knob_dict[key]
            point = [knob_dict[key] for key in knob_dict.keys()]
        return point, valid

    def constrained_crossover_and_mutate(self, m1, m2, keys):
        """Child takes each key variable from either parent, except one mutation key left free
        (knobManager.py:326-339)."""
        known = {}
        if len(keys) > 0:
            midx = random.randint(0, len(keys) - 1)
            for idx, key in enumerate(keys):
                if idx == midx:
                    continue
                known[key] = [m1.solved_knob_vals_genotype[key], m2.solved_knob_vals_genotype[key]]
        try:
            valid, res = self.randSample(known)
        except (AssertionError, RuntimeError):
            # the two parents cannot be combined on these keys (or the search gave up): fall back to a fresh sample
            valid, res = self.randSample({})
        return res, valid

    def onepoint_crossover_and_mutation(self, keys, m1, m2, feasible):
        position = random.randint(0, len(keys) - 1)
        m1_keys = keys[:position]
        known = {}
        mkey = keys[random.randint(0, len(keys) - 1)]
        res = []
        for key in m1.solved_knob_vals_genotype.keys():
            if key == mkey:
                cands = feasible[key]
                known[key] = cands[random.randint(0, len(cands) - 1)]
            elif key in m1_keys:
                known[key] = m1.solved_knob_vals_genotype[key]
            else:
                known[key] = m2.solved_knob_vals_genotype[key]
            res.append(known[key])
        return known, res

    def crossover_and_mutate(self, m1, m2, feasible):
        known, _ = self.onepoint_crossover_and_mutation(self.knob_names, m1, m2, feasible)
        known = {k: known[k] for k in self.knob_names}
        return self.validate(known)

    def crossover_and_mutate_all(self, m1, m2, feasible):
        keys = list(m1.solved_knob_vals_genotype.keys())
        known, res = self.onepoint_crossover_and_mutation(keys, m1, m2, feasible)
        self.solved_knob_vals_genotype = known
        self.solved_knob_vals_phenotype = known
        score = self.solver.SATScore(known)
        self._valid = score == 0
        return res, self._valid, score

    def satdecoding_crossover_and_mutate(self, m1, m2, feasible):
        keys = list(m1.solved_knob_vals_genotype.keys())
        genotype_dict, _ = self.onepoint_crossover_and_mutation(keys, m1, m2, feasible)
        self.solved_knob_vals_genotype = genotype_dict
        valid, phenotype = self.solver.repair(genotype_dict)
        self._valid = valid
        assert valid
        for idx, key in enumerate(list(self.solver.vals.keys())):
            self.solved_knob_vals_phenotype[key] = phenotype[idx]
        return phenotype, valid

    def SBX_crossover_and_mutation(self, m1, m2, feasible, eta_c=15, eta_m=20, p_mut=0.1):
        """Simulated-binary crossover and polynomial mutation over ALL variables, each result snapped to the nearest
        value seen feasible for that variable; the child may violate constraints and carries the per-constraint
        violations for the infeasibility-driven ranking (knobManager.py:392-430)."""
        chrom, res = {}, []
        for key in m1.solved_knob_vals_genotype.keys():
            x1, x2 = m1.solved_knob_vals_genotype[key], m2.solved_knob_vals_genotype[key]
            cands = feasible[key]
            u = random.random()
            if u <= 0.5:
                beta = (2 * u) ** (1.0 / eta_c + 1)
            else:
                beta = (1.0 / (2 * (1 - u + 1e-8))) ** (1.0 / eta_c + 1)
            beta *= random.choice((-1.0, 1.0))
            x = 0.5 * ((1 + beta) * x1 + (1 - beta) * x2)
            x = min(cands, key=lambda t: abs(t - x))
            if random.random() < p_mut:
                span = max(cands) - min(cands)
                r = random.random()
                delta = (2 * r) ** (1.0 / (eta_m + 1)) - 1 if r < 0.5 else 1 - (2 * (1 - r)) ** (1.0 / (eta_m + 1))
                x = min(cands, key=lambda t: abs(t - (x + span * delta)))
            chrom[key] = x
            res.append(x)
        violations, valid = self.solver.MultiSATScore(chrom)
        self.solved_knob_vals_genotype = chrom
        self.solved_knob_vals_phenotype = chrom
        self._valid = valid
        return res, valid, violations

    def constrained_random_walk(self, knob_manager, ratio):
        """Keep a random ``ratio`` of the parent's values, re-solve the rest (knobManager.py:433-444)."""
        keys = list(knob_manager.solved_knob_vals_genotype.keys())
        preserve_num = int(ratio * len(keys))
        positions = set(np.random.choice(len(keys), preserve_num, replace=False).tolist())
        known = {key: [knob_manager.solved_knob_vals_genotype[key]] for idx, key in enumerate(keys) if idx in positions}
        try:
            valid, res = self.randSample(known)
        except RuntimeError:
            valid, res = self.randSample({})        # the search gave up on this subset: a fresh point instead
        return res, valid

    def random_walk(self, knob_manager, feasible):
        knob_name = self.knob_names[random.randint(0, len(self.knob_names) - 1)]
        candidates = feasible[knob_name]
        val = candidates[random.randint(0, len(candidates) - 1)]
        new_knobs = {name: (val if name == knob_name else knob_manager.solved_knob_vals_genotype[name])
                     for name in self.knob_names}
        point = [new_knobs[name] for name in self.knob_names]
        res, valid = self.validate(new_knobs)
        return (res if valid else point), valid

    def valid(self):
        return self._valid
