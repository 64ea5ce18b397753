"""The parts layers are put together from. Importing this package registers them."""
from .base import FixedState, PagedKV, ParamSpec, Part
from . import norm, position, attention, mlp, block, embedding   # noqa: F401  (registration)

__all__ = ["FixedState", "PagedKV", "ParamSpec", "Part"]
