"""Constraint primitives of the schedule CSP.

Same six primitives, argument conventions and dump text as the reference
(schedule/constraints/ortools/primitives.py:13-180), but instead of emitting OR-tools CP-SAT
calls each primitive carries its own finite-domain propagator (``propagate``), used by the
solver in ``solver.py``; OR-tools is not a dependency.

``eval`` returns a violation score that is 0 exactly when the constraint holds.  (The
reference's ``LE.eval``/``LT.eval`` return ``max(b - a, 0)``, which is positive when the
constraint is *satisfied*; here the score is ``max(a - b, 0)`` as the name says.)
"""


import re

_NOT_IDENT = re.compile(r"[^0-9A-Za-z_]")


def removedot(name):
    """Variable name as it appears in a dump: every character that cannot be part of an identifier
    (the dots of split axes, and '#', ':', ',' of generated keys) becomes '_'."""
    if isinstance(name, str):
        return _NOT_IDENT.sub('_', name)
    return name


def getVal(val_dict, v):
    if isinstance(v, str):
        return val_dict[v]
    return int(v)


class _Binary:
    op = '?'

    def __init__(self, args, cond=None):
        assert len(args) == 2
        self.args = list(args)
        self.cond = cond

    def variables(self):
        vs = [a for a in self.args if isinstance(a, str)]
        if self.cond is not None:
            vs.append(self.cond)
        return vs

    def desc(self):
        a, b = removedot(self.args[0]), removedot(self.args[1])
        if self.cond is not None:
            return "model.Add(%s %s %s).OnlyEnforceIf(%s)\n" % (a, self.op, b, removedot(self.cond))
        return "model.Add(%s %s %s)\n" % (a, self.op, b)

    def _active(self, val_dict):
        return self.cond is None or getVal(val_dict, self.cond) == 1

    # --- propagation -------------------------------------------------------------------
    def propagate(self, S):
        """Narrow domains in store S; returns False on a wipe-out."""
        if self.cond is not None:
            c = S.dom(self.cond)
            if c.is_fixed() and c.lo == 0:
                return True
            if not (c.is_fixed() and c.lo == 1):
                # not enforced yet: if the relation is impossible the condition must be 0
                if not self._possible(S):
                    return S.assign(self.cond, 0)
                return True
        return self._enforce(S)


class EQ(_Binary):
    op = '=='

    def eval(self, val_dict):
        if not self._active(val_dict):
            return 0
        return abs(getVal(val_dict, self.args[1]) - getVal(val_dict, self.args[0]))

    def _possible(self, S):
        return S.view(self.args[0]).intersects(S.view(self.args[1]))

    def _enforce(self, S):
        a, b = self.args
        return S.intersect(a, S.view(b)) and S.intersect(b, S.view(a))


class NE(_Binary):
    op = '!='

    def eval(self, val_dict):
        # mirrors the reference: an inactive conditional NE scores 1 (never used conditionally there)
        if self.cond is not None and getVal(val_dict, self.cond) != 1:
            return 1
        return 0 if getVal(val_dict, self.args[0]) != getVal(val_dict, self.args[1]) else 1

    def _possible(self, S):
        a, b = S.view(self.args[0]), S.view(self.args[1])
        return not (a.is_fixed() and b.is_fixed() and a.lo == b.lo)

    def _enforce(self, S):
        a, b = S.view(self.args[0]), S.view(self.args[1])
        if a.is_fixed() and not S.remove(self.args[1], a.lo):
            return False
        if b.is_fixed() and not S.remove(self.args[0], b.lo):
            return False
        return True


class LE(_Binary):
    op = '<='
    strict = 0

    def eval(self, val_dict):
        if not self._active(val_dict):
            return 0
        a, b = getVal(val_dict, self.args[0]), getVal(val_dict, self.args[1])
        return max(a - b + self.strict, 0)

    def _possible(self, S):
        return S.view(self.args[0]).lo + self.strict <= S.view(self.args[1]).hi

    def _enforce(self, S):
        a, b = self.args
        return S.set_max(a, S.view(b).hi - self.strict) and S.set_min(b, S.view(a).lo + self.strict)


class LT(LE):
    op = '<'
    strict = 1


class ProdTwo:
    """args = [target, [a, b]]  meaning  target == a * b  (all values >= 0)."""

    def __init__(self, args):
        assert len(args) == 2 and len(args[1]) == 2
        self.args = [args[0], list(args[1])]
        self.cond = None

    def variables(self):
        return [a for a in [self.args[0]] + self.args[1] if isinstance(a, str)]

    def desc(self):
        t, (a, b) = self.args
        return "model.AddMultiplicationEquality(%s, [%s, %s])\n" % (removedot(t), removedot(a), removedot(b))

    def eval(self, val_dict):
        t, (a, b) = self.args
        return abs(getVal(val_dict, t) - getVal(val_dict, a) * getVal(val_dict, b))

    def propagate(self, S):
        t, (a, b) = self.args
        T, A, Bd = S.view(t), S.view(a), S.view(b)
        # bounds (all domains are non-negative)
        if not (S.set_min(t, A.lo * Bd.lo) and S.set_max(t, A.hi * Bd.hi)):
            return False
        T = S.view(t)
        for x, X, Y in ((a, A, Bd), (b, Bd, A)):
            if Y.hi > 0 and not S.set_min(x, -(-T.lo // Y.hi)):
                return False
            if Y.lo > 0 and not S.set_max(x, T.hi // Y.lo):
                return False
        T, A, Bd = S.view(t), S.view(a), S.view(b)
        # exact support when it is cheap
        if T.is_fixed() and T.lo > 0:
            tv = T.lo
            if not S.filter(a, lambda v: v > 0 and tv % v == 0 and Bd.contains(tv // v)):
                return False
            A = S.view(a)
            if not S.filter(b, lambda v: v > 0 and tv % v == 0 and A.contains(tv // v)):
                return False
        elif A.is_fixed():
            av = A.lo
            if not S.filter(b, lambda v: T.contains(av * v)):
                return False
            if av > 0 and not S.filter(t, lambda v: v % av == 0 and S.view(b).contains(v // av)):
                return False
        elif Bd.is_fixed():
            bv = Bd.lo
            if not S.filter(a, lambda v: T.contains(bv * v)):
                return False
            if bv > 0 and not S.filter(t, lambda v: v % bv == 0 and S.view(a).contains(v // bv)):
                return False
        elif A.size() * Bd.size() <= 4096:
            prods = set()
            bvals = list(Bd.values())
            for av in A.values():
                for bv in bvals:
                    prods.add(av * bv)
            if not S.filter(t, lambda v: v in prods):
                return False
            T = S.view(t)
            if not S.filter(a, lambda v: any(T.contains(v * bv) for bv in bvals)):
                return False
            avals = list(S.view(a).values())
            if not S.filter(b, lambda v: any(T.contains(av * v) for av in avals)):
                return False
        return True


class Sum:
    """args = [target, [x0, x1, ...]]  meaning  target == sum(xs)."""

    def __init__(self, args):
        assert len(args) == 2
        self.args = [args[0], list(args[1])]
        self.cond = None

    def variables(self):
        return [a for a in [self.args[0]] + self.args[1] if isinstance(a, str)]

    def desc(self):
        t, xs = self.args
        return "model.Add(sum([%s]) == %s)\n" % (", ".join(str(removedot(x)) for x in xs), removedot(t))

    def eval(self, val_dict):
        t, xs = self.args
        return abs(getVal(val_dict, t) - sum(getVal(val_dict, x) for x in xs))

    def propagate(self, S):
        t, xs = self.args
        views = [S.view(x) for x in xs]
        lo, hi = sum(v.lo for v in views), sum(v.hi for v in views)
        if not (S.set_min(t, lo) and S.set_max(t, hi)):
            return False
        T = S.view(t)
        for x, v in zip(xs, views):
            # x = t - (sum of the others)
            if not (S.set_min(x, T.lo - (hi - v.hi)) and S.set_max(x, T.hi - (lo - v.lo))):
                return False
        return True
