from .context import Context
from .cdna_context import CDNA4Context, GFX950_LIMITS


def buildContext(_type, knob_manager, build_kwargs, target_name):
    """Dispatch by codegen type, as schedule/context/__init__.py:5-15 of the reference does."""
    if _type == 'GPU_MFMA':
        return CDNA4Context(knob_manager, build_kwargs, target_name)
    raise ValueError('Unsupportted code gen type %s' % _type)
