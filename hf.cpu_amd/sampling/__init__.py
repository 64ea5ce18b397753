"""Sampling: the reference's random numbers and pipeline; whole-vocabulary work on the GPU."""
from .rng import Rng
from .sampler import Choice, Sampler, SamplerParams

__all__ = ["Choice", "Rng", "Sampler", "SamplerParams"]
