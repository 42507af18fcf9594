"""One point of the search space (sample.py:8-27 of the reference)."""
import copy

from .utils import DeCode


class Sample:
    def __init__(self, task):
        self.valid = False
        self.perf = 0.0
        self.task = task
        self.knob_manager = copy.deepcopy(task.knob_manager)
        self.predict = 0
        self.prob = 0
        self.violation = None
        self.violations = None
        self.ranks = []
        self.point = None
        self.stmt_code = None

    def getTask(self):
        return self.task

    def fromCode(self, code):
        point = DeCode(code)
        self.point = point
        for idx, key in enumerate(list(self.knob_manager.solver.vals.keys())):
            self.knob_manager.solved_knob_vals_genotype[key] = point[idx]
            self.knob_manager.solved_knob_vals_phenotype[key] = point[idx]

    def lower(self):
        return self.getTask().getStmt(self.knob_manager)
