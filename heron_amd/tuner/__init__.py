from .tuner import Tuner  # noqa: F401
from .ga_tuner import CGATuner, GATuner, RCGATuner  # noqa: F401
from .random_tuner import CRandSampler, CRandTuner  # noqa: F401
