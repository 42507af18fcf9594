from .knobManager import KnobManager  # noqa: F401
from .solver import Solver, Variable  # noqa: F401
from .primitives import EQ, LE, LT, NE, ProdTwo, Sum  # noqa: F401
