"""The step function and what drives it."""
from .batch import Entry, StepInputs
from .engine import Engine

__all__ = ["Engine", "Entry", "StepInputs"]
