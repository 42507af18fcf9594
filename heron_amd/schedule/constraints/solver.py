"""Finite-domain solver for the schedule CSP (no OR-tools).

Interface of the reference's ``Solver`` (schedule/constraints/ortools/solver.py:18-177):
``addVal``, ``vals``, ``primitives``, ``solve(hint, known, bounds)``, ``validate``, ``repair``,
``SATScore``, ``MultiSATScore``, ``dump``.  Where the reference builds a CP-SAT model with
shuffled variable/constraint order and takes the first feasible point, this solver runs
domain propagation (each primitive narrows the domains it touches, to a fixpoint) plus a
randomised depth-first search: hinted variables are branched first, hint value first, the
other values and variables in random order; a fail budget triggers a restart with a new order.
"""
import random
import re

from .primitives import EQ, LE, LT, NE, ProdTwo, Sum, removedot

ENUM_LIMIT = 1 << 14     # domains up to this size are held as explicit value sets


class Variable:
    def __init__(self, name, low, up, item, defv):
        self.low = low
        self.up = up
        self.item = item
        self.defv = defv
        self.name = name

    def __repr__(self):
        return "Var(%s, %d, %d, %d)" % (self.name, self.low, self.up, self.defv)


class Domain:
    """Immutable integer domain: an interval, optionally restricted to an explicit value set."""
    __slots__ = ("lo", "hi", "vals")

    def __init__(self, lo, hi, vals=None):
        self.lo, self.hi, self.vals = lo, hi, vals

    @staticmethod
    def make(lo, hi):
        if hi - lo + 1 <= ENUM_LIMIT:
            return Domain(lo, hi, frozenset(range(lo, hi + 1)))
        return Domain(lo, hi, None)

    @staticmethod
    def of(values):
        vs = frozenset(values)
        return Domain(min(vs), max(vs), vs) if vs else None

    def is_fixed(self):
        return self.lo == self.hi

    def size(self):
        return len(self.vals) if self.vals is not None else self.hi - self.lo + 1

    def contains(self, v):
        if v < self.lo or v > self.hi:
            return False
        return self.vals is None or v in self.vals

    def values(self):
        return sorted(self.vals) if self.vals is not None else range(self.lo, self.hi + 1)

    def intersects(self, o):
        if self.hi < o.lo or o.hi < self.lo:
            return False
        if self.vals is not None and o.vals is not None:
            small, big = (self.vals, o.vals) if len(self.vals) <= len(o.vals) else (o.vals, self.vals)
            return any(v in big for v in small)
        if self.vals is not None:
            return any(o.lo <= v <= o.hi for v in self.vals)
        if o.vals is not None:
            return any(self.lo <= v <= self.hi for v in o.vals)
        return True

    def narrowed(self, lo=None, hi=None, keep=None):
        """A new domain (or None when empty); returns self when nothing changes."""
        nlo = self.lo if lo is None else max(self.lo, lo)
        nhi = self.hi if hi is None else min(self.hi, hi)
        if nlo > nhi:
            return None
        if self.vals is None:
            if keep is None:
                if nlo == self.lo and nhi == self.hi:
                    return self
                if nhi - nlo + 1 <= ENUM_LIMIT:
                    return Domain(nlo, nhi, frozenset(range(nlo, nhi + 1)))
                return Domain(nlo, nhi, None)
            if nhi - nlo + 1 > ENUM_LIMIT:             # too wide to filter value by value yet
                return self if (nlo == self.lo and nhi == self.hi) else Domain(nlo, nhi, None)
            vs = frozenset(v for v in range(nlo, nhi + 1) if keep(v))
        else:
            if keep is None and nlo == self.lo and nhi == self.hi:
                return self
            if keep is None:
                vs = frozenset(v for v in self.vals if nlo <= v <= nhi)
            else:
                vs = frozenset(v for v in self.vals if nlo <= v <= nhi and keep(v))
            if len(vs) == len(self.vals):
                return self
        if not vs:
            return None
        return Domain(min(vs), max(vs), vs)


class Store:
    """Domains of all variables during one search, with change notification."""

    def __init__(self, doms, watchers):
        self.doms = doms
        self.watchers = watchers
        self.queue = []
        self.queued = set()

    def copy(self):
        return Store(dict(self.doms), self.watchers)

    def dom(self, name):
        return self.doms[name]

    def view(self, x):
        if isinstance(x, str):
            return self.doms[x]
        x = int(x)
        return Domain(x, x, frozenset((x,)))

    def _update(self, name, nd):
        if nd is None:
            return False
        if nd is not self.doms[name]:
            self.doms[name] = nd
            for ci in self.watchers.get(name, ()):
                if ci not in self.queued:
                    self.queued.add(ci)
                    self.queue.append(ci)
        return True

    def set_min(self, x, lo):
        if not isinstance(x, str):
            return int(x) >= lo
        return self._update(x, self.doms[x].narrowed(lo=lo))

    def set_max(self, x, hi):
        if not isinstance(x, str):
            return int(x) <= hi
        return self._update(x, self.doms[x].narrowed(hi=hi))

    def assign(self, x, v):
        if not isinstance(x, str):
            return int(x) == v
        d = self.doms[x]
        if not d.contains(v):
            return False
        return self._update(x, Domain(v, v, frozenset((v,))))

    def remove(self, x, v):
        if not isinstance(x, str):
            return int(x) != v
        d = self.doms[x]
        if not d.contains(v):
            return True
        if d.vals is None:
            if v == d.lo:
                return self._update(x, d.narrowed(lo=v + 1))
            if v == d.hi:
                return self._update(x, d.narrowed(hi=v - 1))
            return True
        return self._update(x, d.narrowed(keep=lambda u: u != v))

    def filter(self, x, keep):
        if not isinstance(x, str):
            return bool(keep(int(x)))
        return self._update(x, self.doms[x].narrowed(keep=keep))

    def intersect(self, x, other):
        if not isinstance(x, str):
            return other.contains(int(x))
        d = self.doms[x]
        if other.vals is not None:
            return self._update(x, d.narrowed(lo=other.lo, hi=other.hi, keep=lambda v: v in other.vals))
        return self._update(x, d.narrowed(lo=other.lo, hi=other.hi))


class Solver:
    def __init__(self):
        self.vals = {}
        self.primitives = []
        self.fail_budget = 400
        self.restarts = 8
        self.last_status = None         # 'feasible' | 'infeasible' | 'unknown' of the last solve
        self.budget_hits = 0            # searches given up on their fail budget since construction
        self._budget_hit = False
        self._sampled_out = False

    def addVal(self, name, low, up, def_val):
        assert name not in self.vals.keys()
        self.vals[name] = Variable(name, low, up, None, def_val)

    def getVal(self, v):
        if isinstance(v, str):
            assert v in self.vals.keys()
            return self.vals[v].item
        return int(v)

    # ------------------------------------------------------------------ search machinery
    def _watchers(self):
        w = {}
        for ci, p in enumerate(self.primitives):
            for v in p.variables():
                w.setdefault(v, []).append(ci)
        return w

    def _fixpoint(self, S, initial=None):
        if initial is not None:
            for ci in initial:
                if ci not in S.queued:
                    S.queued.add(ci)
                    S.queue.append(ci)
        while S.queue:
            ci = S.queue.pop()
            S.queued.discard(ci)
            if not self.primitives[ci].propagate(S):
                S.queue.clear()
                S.queued.clear()
                return False
        return True

    def _root(self, known, bounds, fixed=None):
        doms = {}
        for key, v in self.vals.items():
            lo, hi = v.low, v.up
            if key in bounds:
                lo, hi = max(lo, bounds[key][0]), min(hi, bounds[key][1])
            if lo > hi:
                return None
            doms[key] = Domain.make(lo, hi)
        S = Store(doms, self._watchers())
        for key, cands in known.items():
            cands = list(cands) if isinstance(cands, (list, tuple, set)) else [cands]
            assert 1 <= len(cands) <= 2, "known takes one value or a pair (crossover)"
            cs = set(int(c) for c in cands)
            if not S.filter(key, lambda v: v in cs):
                return None
        if fixed:
            for key, val in fixed.items():
                if key in doms and not S.assign(key, int(val)):
                    return None
        if not self._fixpoint(S, range(len(self.primitives))):
            return None
        return S

    @staticmethod
    def _candidates(d, hint, rng):
        if d.vals is not None:
            vals = list(d.vals)
            rng.shuffle(vals)
        else:
            vals = [d.lo, d.hi] + [rng.randint(d.lo, d.hi) for _ in range(6)]
        if hint is not None and d.contains(hint):
            vals = [hint] + [v for v in vals if v != hint]
        return vals

    def _search(self, root, hint, rng):
        names = list(self.vals.keys())
        hinted = [k for k in names if k in hint]
        others = [k for k in names if k not in hint]
        rng.shuffle(hinted)
        rng.shuffle(others)
        order = hinted + others
        fails = 0
        # explicit stack of (store, position in order, remaining values)
        stack = []
        S, pos = root, 0
        while True:
            while pos < len(order) and S.doms[order[pos]].is_fixed():
                pos += 1
            if pos == len(order):
                return [S.doms[k].lo for k in names]
            var = order[pos]
            stack.append((S, pos, self._candidates(S.doms[var], hint.get(var), rng)))
            advanced = False
            while stack:
                S0, pos0, cands = stack[-1]
                if not cands:
                    d0 = S0.doms[order[pos0]]
                    if d0.vals is None and d0.hi - d0.lo + 1 > 8:
                        self._sampled_out = True        # an interval was only sampled: nothing is proven
                    stack.pop()
                    continue
                v = cands.pop(0)
                S1 = S0.copy()
                if S1.assign(order[pos0], v) and self._fixpoint(S1):
                    S, pos = S1, pos0 + 1
                    advanced = True
                    break
                fails += 1
                if fails > self.fail_budget:
                    self._budget_hit = True
                    return None
            if not advanced:
                return None

    def _solve(self, hint, known, bounds, fixed=None, rng=None):
        """(valid, point).  ``self.last_status`` says which kind of "not valid" it was: 'infeasible' (propagation or an
        exhausted search proved that no point exists) or 'unknown' (every restart ran out of its fail budget; the
        system may still be feasible - the reference's CP-SAT is complete and never reports this)."""
        rng = rng or random
        self.last_status = 'infeasible'
        root = self._root(known, bounds, fixed)
        if root is None:
            return False, None
        budget = self.fail_budget
        try:
            for attempt in range(self.restarts + 1):
                if attempt == self.restarts:
                    # last resort: one search with a budget large enough to settle most systems either way
                    self.fail_budget = budget * 25
                self._budget_hit = self._sampled_out = False
                res = self._search(root, hint, rng)
                if res is not None:
                    self.last_status = 'feasible'
                    return True, res
                if not self._budget_hit and not self._sampled_out:
                    return False, None          # the search space was exhausted: proven infeasible
                self.budget_hits += 1
        finally:
            self.fail_budget = budget
        self.last_status = 'unknown'
        return False, None

    # ------------------------------------------------------------------ reference interface
    def solve(self, hint, known, bounds={}):
        """First feasible point reached from random orders, preferring ``hint`` values.

        ``known[key]`` is a list of one value (fixed) or two values (crossover: either parent's),
        ``bounds[key] = [low, up]`` narrows a variable.  Returns ``(valid, values in definition order)``.
        """
        return self._solve(hint, known, bounds)

    def validate(self, knob_dict):
        """Is there a full assignment that extends ``knob_dict``?"""
        for k, v in knob_dict.items():
            if k in self.vals and not (self.vals[k].low <= v <= self.vals[k].up):
                return False, None
        return self._solve({}, {}, {}, fixed=knob_dict)

    def repair(self, val_dict):
        """A feasible point near ``val_dict`` (every entry is used as a hint)."""
        return self._solve(dict(val_dict), {}, {})

    def SATScore(self, val_dict):
        return sum(p.eval(val_dict) for p in self.primitives)

    def MultiSATScore(self, val_dict):
        scores = [p.eval(val_dict) for p in self.primitives]
        return scores, all(s == 0 for s in scores)

    def in_bounds(self, val_dict):
        return all(v.low <= val_dict[k] <= v.up for k, v in self.vals.items())

    def dump(self):
        """Text dump in the format of the reference's constraints.py (solver.py:76-89)."""
        strs = "from ortools.sat.python import cp_model\n\n"
        strs += "model = cp_model.CpModel()\n"
        for key, v in self.vals.items():
            strs += '%s = model.NewIntVar(%d, %d, \'%s\')\n' % (removedot(key), v.low, v.up, removedot(key))
        for p in self.primitives:
            strs += p.desc()
        strs += "solver = cp_model.CpSolver()\n"
        strs += "status = solver.Solve(model)\n"
        return strs

    # ------------------------------------------------------------------ (de)serialisation
    def to_spec(self):
        cons = []
        for p in self.primitives:
            kind = type(p).__name__
            cons.append([kind, p.args, p.cond])
        return {"vars": [[k, v.low, v.up, v.defv] for k, v in self.vals.items()], "cons": cons}

    @classmethod
    def from_spec(cls, spec):
        s = cls()
        for item in spec["vars"]:
            name, lo, hi = item[0], item[1], item[2]
            s.addVal(name, lo, hi, item[3] if len(item) > 3 else lo)
        kinds = {"EQ": EQ, "NE": NE, "LE": LE, "LT": LT}
        for kind, args, cond in spec["cons"]:
            if kind == "ProdTwo":
                s.primitives.append(ProdTwo(args))
            elif kind == "Sum":
                s.primitives.append(Sum(args))
            else:
                s.primitives.append(kinds[kind](args, cond=cond))
        return s

    @classmethod
    def from_dump(cls, text):
        """Parse a constraints.py dump (variables, Add, AddMultiplicationEquality, sum) back into a solver."""
        s = cls()

        def tok(t):
            t = t.strip()
            return int(t) if re.fullmatch(r"-?\d+", t) else t

        ops = {"==": EQ, "!=": NE, "<=": LE, "<": LT}
        for line in text.splitlines():
            line = line.strip()
            m = re.fullmatch(r"(\w+) = model\.NewIntVar\((-?\d+), (-?\d+), '(\w+)'\)", line)
            if m:
                s.addVal(m.group(4), int(m.group(2)), int(m.group(3)), int(m.group(2)))
                continue
            m = re.fullmatch(r"model\.AddMultiplicationEquality\((\w+), \[(\w+), (\w+)\]\)", line)
            if m:
                s.primitives.append(ProdTwo([tok(m.group(1)), [tok(m.group(2)), tok(m.group(3))]]))
                continue
            m = re.fullmatch(r"model\.Add\(sum\(\[(.*)\]\) == (\w+)\)", line)
            if m:
                s.primitives.append(Sum([tok(m.group(2)), [tok(x) for x in m.group(1).split(",")]]))
                continue
            m = re.fullmatch(r"model\.Add\((\w+) (==|!=|<=|<) (-?\w+)\)(?:\.OnlyEnforceIf\((\w+)\))?", line)
            if m:
                s.primitives.append(ops[m.group(2)]([tok(m.group(1)), tok(m.group(3))], cond=m.group(4)))
                continue
        return s
