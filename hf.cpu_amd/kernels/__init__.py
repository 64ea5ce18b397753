"""The hand-written gfx950 kernels: build, load, and call."""
from .lib import load_extension
from .ops import Ops

__all__ = ["Ops", "load_extension"]
