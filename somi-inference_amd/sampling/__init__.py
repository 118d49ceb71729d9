"""Sampling options, the counter-based random stream and the sampler."""

from .params import SamplingParams
from .rng import uniform
from .sampler import Sampler

__all__ = ["Sampler", "SamplingParams", "uniform"]
