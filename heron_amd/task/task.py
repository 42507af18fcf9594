"""Task: one operator instance to tune.

Keeps the interface of the reference's task/task.py:13-103 - ``make_stage_schedules`` (build the template and its
constraint system), ``instantiate`` (replay the recorded schedule steps with a solved KnobManager into a concrete
template instance), ``apply_best`` (the best row of a records file), ``apply_sample``, ``set_verify_func`` (arms the
measurer's result check), ``getStmt`` - on top of a fixed HIP template instead of TVM loop nests.
"""
import json
import os

from ..schedule.constraints import KnobManager
from ..schedule.context import buildContext
from ..schedule.sched_op import TemplateSchedule, get_op_methods, sched_via_rule


class Task:
    def __init__(self, name, opfunc, args, target, target_host=None):
        self.name, self.opfunc, self.args = name, opfunc, args
        self.target, self.target_host = target, target_host
        self.config = None
        self.build_kwargs = None
        self.device_id = 0
        self.knob_manager = KnobManager()
        self.sched_desc = ""
        self.template_info = None           # operator / element kind / GEMM view, known once the template is built
        # result check of the measurer (off until set_verify_func is called, as in the reference)
        self.not_verify_correctness = True
        self.ref_input = self.ref_output = None
        self.rtol = 0.1

    def code(self):
        return self.name

    # ------------------------------------------------------------------ template and constraint system
    def _declare(self, knob_manager):
        """Runs the operator definition under a fresh context; returns (context, schedule object, output tensors)."""
        ctx = buildContext(self.config.codegen_type, knob_manager, self.build_kwargs, str(self.target))
        outs = self.opfunc(ctx, *self.args)
        sched = TemplateSchedule(outs, ctx.tensorize_info)
        ctx.init_tensor_dict(outs)
        return ctx, sched, outs

    def getOut(self):
        return self._declare(self.knob_manager)[2]

    def make_stage_schedules(self):
        print(self.args)
        ctx, sched, _ = self._declare(self.knob_manager)
        sched_via_rule(self.config.codegen_type, ctx, sched)
        self.sched_desc = ctx.sched_desc
        self.template_info = ctx.tensorize_info
        self.knob_manager.is_building = False
        solver = self.knob_manager.solver
        feasible, _ = solver.solve({}, {})
        for _ in range(4):
            if feasible or solver.last_status != 'unknown':
                break
            feasible, _ = solver.solve({}, {})      # the randomised search gave up; that proves nothing
        self.dump_constraints()
        if not feasible:
            raise AssertionError("the template has no feasible instance for this shape (solver: %s)" % solver.last_status)

    def dump_constraints(self):
        log_dir = getattr(self.config, "log_dir", None)
        if log_dir and os.path.isdir(log_dir):
            with open(os.path.join(log_dir, 'constraints.py'), 'w') as out:
                out.write(self.knob_manager.solver.dump())

    def instantiate(self, knob_manager):
        """(template schedule, argument tensors) of the point ``knob_manager`` holds."""
        ctx, sched, outs = self._declare(knob_manager)
        methods = get_op_methods(self.config.codegen_type)
        for action, stage in knob_manager.sched_tups:
            methods[action](action).perform(sched, stage, ctx)
        ctx.pos_process(sched)
        knob_manager.sched_desc = ctx.sched_desc
        return sched, ctx.input_tensors + outs

    # ------------------------------------------------------------------ points from records and samples
    def _instantiate_values(self, values, perf):
        km = self.knob_manager
        km.solved_knob_vals_phenotype = values
        km.runtime_perf = perf
        km.is_building = False
        return self.instantiate(km)

    @staticmethod
    def best_record(path):
        """The row of a records file that ships: the best of the rows re-timed with long repeats at the end of a
        search ("confirmed": true) when there are any, else the best row (the reference's rule, task/task.py:30-43)."""
        rows = [json.loads(line) for line in open(path) if line.strip()]
        confirmed = [r for r in rows if r.get('confirmed') and r['perf'] != 0]
        return max(confirmed or rows, key=lambda r: r['perf'])

    def apply_best(self, path):
        """Instantiates the best-performing row of a records file."""
        if not self.knob_manager.sched_tups:
            self.make_stage_schedules()
        best = self.best_record(path)
        # a record written before a knob was added to the template lacks that knob: it then takes its default
        values = {name: var.defv for name, var in self.knob_manager.solver.vals.items()}
        values.update(best['param'])
        return self._instantiate_values(values, best['perf'])

    def apply_sample(self, sample):
        """Instantiates a measured sample (the reference's version reads an undefined name, task/task.py:45-49)."""
        return self._instantiate_values(dict(sample.knob_manager.solved_knob_vals_phenotype), sample.perf)

    # ------------------------------------------------------------------ cost-model features
    def featurize(self, values, own_shape=True):
        """Compact feature vector of a solved point, or None when the operator set defines none.  ``own_shape=False``:
        the point belongs to another task of the same operator (a record of an earlier run) and is described with
        that task's extents."""
        if self.template_info is None or self.config is None or self.config.codegen_type != 'GPU_MFMA':
            return None
        from ..schedule.sched_op.mfma_features import featurize, view_of_values
        info = self.template_info if own_shape else view_of_values(self.template_info, values)
        return featurize(info, values)

    def coupled_moves(self, knob_manager):
        """(label, knob dictionary) pairs a few coordinated knob changes away from the point ``knob_manager`` holds
        (operator specific; empty when the operator set defines none); moves that share a label differ only in dependent
        choices.  Used by the refinement rounds and the confirmation phase of the search."""
        if self.template_info is None or self.config is None or self.config.codegen_type != 'GPU_MFMA':
            return []
        from ..schedule.sched_op.mfma_features import coupled_moves
        names = list(knob_manager.knob_names)
        values = {n: knob_manager.solved_knob_vals_genotype[n] for n in names}
        return coupled_moves(names, values, knob_manager.get_knob_candidates)

    # ------------------------------------------------------------------ verification and text form
    def set_verify_func(self, func, rtol=0.1):
        self.rtol = rtol
        self.not_verify_correctness = False
        print("Caculating on cpu to verify correctness")
        self.ref_input, self.ref_output = func(self.args)
        print("End")

    def getStmt(self, knob_manager):
        """Text form of an instance (the reference returns the lowered TIR here)."""
        sched, args = self.instantiate(knob_manager)
        lines = ["%s %s" % (sched.info['operator'], sched.info['kind'])]
        lines += ["  %s: %s %s" % (t.name, t.shape, t.dtype) for t in args]
        lines.append("  template: " + sched.describe())
        return "\n".join(lines)
