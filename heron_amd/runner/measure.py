"""Measurement records and the build->run batch function.

Own equivalents of the autotvm types the reference imports (``MeasureInput``, ``MeasureResult``,
``MeasureErrorNo``, ``measure_option``, ``create_measure_batch``; used at environment.py:35,110-120
and runner/runner.py:28-29).
"""
from collections import namedtuple


class MeasureInput(namedtuple("MeasureInput", ["target", "task", "config"])):
    """target string, the Task, and the solved KnobManager of one sample."""


class MeasureResult(namedtuple("MeasureResult", ["costs", "error_no", "all_cost", "timestamp"])):
    """costs: seconds (or error objects), error_no: MeasureErrorNo, all_cost: wall seconds spent."""


class MeasureErrorNo(object):
    NO_ERROR = 0
    INSTANTIATION_ERROR = 1
    COMPILE_HOST = 2
    COMPILE_DEVICE = 3
    RUNTIME_DEVICE = 4
    WRONG_ANSWER = 5
    BUILD_TIMEOUT = 6
    RUN_TIMEOUT = 7
    UNKNOWN_ERROR = 8
    # the reference's measurer reports a failed result check as the bare number 100
    # (runner/measure_methods.py:176-177)
    VERIFY_FAILED = 100


# ``adapter``: the operator's info dictionary when its operands go through an operand adapter (then the pre-stage is
# part of what gets timed), None for operators that hand their tensors to the kernel as they are
BuildResult = namedtuple("BuildResult", ["desc_tuple", "problem", "arg_info", "error", "time_cost", "adapter"],
                         defaults=(None,))


def measure_option(builder, runner):
    return {"builder": builder, "runner": runner}


def create_measure_batch(task, option):
    builder, runner = option["builder"], option["runner"]
    attach_objects = runner.set_task(task)
    build_kwargs = runner.get_build_kwargs()
    builder.set_task(task, build_kwargs)

    def measure_batch(measure_inputs):
        build_results = builder.build(measure_inputs)
        return runner.run(measure_inputs, build_results)

    measure_batch.n_parallel = builder.n_parallel
    measure_batch.attach_objects = attach_objects
    return measure_batch
