"""One point of a task's search space: a private copy of the task's KnobManager (solved values live there), the
point as a flat vector of every solver variable in definition order (``point``), its text form (``stmt_code``) and the
bookkeeping the tuners attach (prediction, measured perf, constraint violations).  Counterpart of the reference's
sample.py:8-27, without the TVM lowering."""
import copy

from .utils import DeCode


class Sample:
    def __init__(self, task):
        self.task = task
        self.knob_manager = copy.deepcopy(task.knob_manager)
        self.point = None
        self.stmt_code = None
        self.valid = False
        self.perf = 0.0
        self.predict = 0
        self.prob = 0
        self.violation = None           # total constraint violation (stochastic ranking)
        self.violations = None          # per-constraint violations (IDEA)
        self.ranks = []

    def getTask(self):
        return self.task

    def values(self):
        """name -> value of every solver variable of this point."""
        return self.knob_manager.solved_knob_vals_phenotype

    def features(self):
        """What the cost model sees: the task's compact feature vector when its operator set defines one, else the
        raw point (the reference's choice, tuner/tuner.py:322-323)."""
        f = self.task.featurize(self.values()) if hasattr(self.task, "featurize") else None
        return list(self.point) if f is None else f

    def prior(self):
        """ln(1 / estimated seconds) from the task's analytic model (the last feature), None when there is none."""
        f = self.task.featurize(self.values()) if hasattr(self.task, "featurize") else None
        return None if f is None else f[-1]

    def fromCode(self, code):
        """Restores the point from its text form."""
        self.point = DeCode(code)
        self.stmt_code = code
        for name, value in zip(self.knob_manager.solver.vals, self.point):
            self.knob_manager.solved_knob_vals_genotype[name] = value
            self.knob_manager.solved_knob_vals_phenotype[name] = value
