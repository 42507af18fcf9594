"""CPU oracle for the Heron hot path - test infrastructure, never part of the product path.

Only the tests, the smoke check and the benchmark's ``cpu_baseline`` leg import this package.
"""
from .ref import *  # noqa: F401,F403
