"""The hand-written gfx950 kernels: build, load, and call."""
from .ops import Ops

__all__ = ["Ops"]
