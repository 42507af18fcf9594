from .measure import MeasureErrorNo, MeasureInput, MeasureResult, create_measure_batch, measure_option  # noqa: F401
from .measure_methods import HipBuilder, HipRunner, LocalBuilder, LocalRunner  # noqa: F401
from .runner import Runner  # noqa: F401
