from .tuner import Tuner  # noqa: F401
from .ga_tuner import CGATuner, GATuner, RCGATuner, SDGATuner, SRGATuner  # noqa: F401
from .idea_tuner import IDEATuner  # noqa: F401
from .sa_tuner import ConstrainedRandomWalkerSATuner, RandomWalkSATuner, SATuner  # noqa: F401
from .random_tuner import CRandSampler, CRandTuner  # noqa: F401
