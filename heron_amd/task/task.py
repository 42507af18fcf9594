"""Task: one operator instance to tune - API of the reference's task/task.py:13-103.

``make_stage_schedules`` builds the template and its constraint system, ``instantiate`` replays
the recorded schedule steps with a solved KnobManager into a concrete template instance,
``apply_best`` loads the best row of a records file, ``set_verify_func`` arms the result check
of the measurer.
"""
import json
import os

from ..schedule.constraints import KnobManager
from ..schedule.context import buildContext
from ..schedule.sched_op import TemplateSchedule, get_op_methods, sched_via_rule


class Task:
    def __init__(self, name, opfunc, args, target, target_host=None):
        self.name = name
        self.args = args
        self.opfunc = opfunc
        self.target = target
        self.target_host = target_host
        self.build_kwargs = None
        self.knob_manager = KnobManager()
        self.not_verify_correctness = True
        self.ref_input = None
        self.ref_output = None
        self.rtol = 0.1
        self.config = None
        self.device_id = 0
        self.sched_desc = ""

    def code(self):
        return self.name

    def _context(self, knob_manager):
        return buildContext(self.config.codegen_type, knob_manager, self.build_kwargs, str(self.target))

    def apply_best(self, path):
        if self.knob_manager.sched_tups == []:
            self.make_stage_schedules()
        to_sort = []
        for row in open(path):
            if not row.strip():
                continue
            json_dict = json.loads(row)
            to_sort.append((json_dict['perf'], json_dict['param']))
        sorted_pairs = sorted(to_sort, key=lambda x: -x[0])
        # a record written before a knob was added to the template lacks that knob: it then takes its default (off)
        param = {name: var.defv for name, var in self.knob_manager.solver.vals.items()}
        param.update(sorted_pairs[0][1])
        self.knob_manager.solved_knob_vals_phenotype = param
        self.knob_manager.runtime_perf = sorted_pairs[0][0]
        self.knob_manager.is_building = False
        return self.instantiate(self.knob_manager)

    def apply_sample(self, sample):
        """Instantiate from a measured sample (the reference's version reads an undefined name)."""
        self.knob_manager.solved_knob_vals_phenotype = dict(sample.knob_manager.solved_knob_vals_phenotype)
        self.knob_manager.runtime_perf = sample.perf
        self.knob_manager.is_building = False
        return self.instantiate(self.knob_manager)

    def getOut(self):
        ctx = self._context(self.knob_manager)
        return self.opfunc(ctx, *self.args)

    def make_stage_schedules(self):
        ctx = self._context(self.knob_manager)
        print(self.args)
        outs = self.opfunc(ctx, *self.args)
        s = TemplateSchedule(outs, ctx.tensorize_info)
        ctx.init_tensor_dict(outs)
        sched_via_rule(self.config.codegen_type, ctx, s)
        self.sched_desc = ctx.sched_desc
        self.knob_manager.is_building = False
        valid, _ = self.knob_manager.solver.solve({}, {})
        self.dump_constraints()
        assert valid, "the template has no feasible instance for this shape"

    def dump_constraints(self):
        log_dir = getattr(self.config, "log_dir", None)
        if not log_dir or not os.path.isdir(log_dir):
            return
        with open(os.path.join(log_dir, 'constraints.py'), 'w') as f:
            f.write(self.knob_manager.solver.dump())

    def instantiate(self, knob_manager):
        ctx = self._context(knob_manager)
        outs = self.opfunc(ctx, *self.args)
        s = TemplateSchedule(outs, ctx.tensorize_info)
        ctx.init_tensor_dict(outs)
        args = ctx.input_tensors + outs
        op_methods = get_op_methods(self.config.codegen_type)
        for act_name, stage_name in knob_manager.sched_tups:
            op_methods[act_name](act_name).perform(s, stage_name, ctx)
        ctx.pos_process(s)
        knob_manager.sched_desc = ctx.sched_desc
        return s, args

    def set_verify_func(self, func, rtol=0.1):
        self.rtol = rtol
        self.not_verify_correctness = False
        print("Caculating on cpu to verify correctness")
        self.ref_input, self.ref_output = func(self.args)
        print("End")

    def getStmt(self, knob_manager):
        """Text form of an instance (the reference returns the lowered TIR here)."""
        s, args = self.instantiate(knob_manager)
        lines = ["%s %s" % (s.info['operator'], s.info['kind'])]
        lines += ["  %s: %s %s" % (t.name, t.shape, t.dtype) for t in args]
        lines.append("  template: " + s.describe())
        return "\n".join(lines)
