from .mfma_operator import all_op_methods as mfma_methods
from .mfma_operator import sched_via_rule as mfma_sched
from .mfma_operator import TemplateSchedule  # noqa: F401

supportted_codegen_types = ['GPU_MFMA']


def get_op_methods(_type):
    """schedule/sched_op/__init__.py:12-23 of the reference, with the one code generator of this backend."""
    if _type == 'GPU_MFMA':
        return mfma_methods
    raise ValueError('Only support ', supportted_codegen_types)


def sched_via_rule(_type, ctx, s):
    if _type == 'GPU_MFMA':
        return mfma_sched(ctx, s)
    raise ValueError('Only support ', supportted_codegen_types)
