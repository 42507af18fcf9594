"""Schedule context: bookkeeping shared by operator definitions and schedule operations.

Keeps the parts of the reference's Context (schedule/context/context.py:7-90) that do not depend
on TVM: the textual schedule description, the replay list ``knob_manager.sched_tups`` filled by
``addSched``, the operator ``info``/``axis_map`` and the tensor dictionary.
"""


class Context:
    def __init__(self, knob_manager, build_kwargs, target_name):
        self.sched_desc = ""
        self.codegen_type = None
        self.target_name = target_name
        self.build_kwargs = build_kwargs
        self.tensor_dict = {}
        self.input_tensors = []
        self.axis_map = {}
        self.tensorize_info = None
        self.knob_manager = knob_manager

    def init_tensor_dict(self, outs):
        for tensor in outs:
            self.tensor_dict[tensor.name] = tensor
            ins = tensor.op.input_tensors
            if len(ins) == 0 and tensor not in self.input_tensors:
                self.input_tensors.append(tensor)
            self.init_tensor_dict(ins)

    def set_info(self, info):
        self.tensorize_info = info

    def set_axis_map(self, axis_map):
        self.axis_map = axis_map

    def addSchedDesc(self, strs, add2Solver=False):
        self.sched_desc += strs

    def pos_process(self, s):
        pass

    def addSched(self, op_name, stage_name, s):
        """Record the step for later replay, then perform it (context.py:68-72)."""
        from ..sched_op import get_op_methods
        self.knob_manager.sched_tups.append((op_name, stage_name))
        action = get_op_methods(self.codegen_type)[op_name](op_name)
        action.perform(s, stage_name, self)
