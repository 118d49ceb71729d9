"""Sampling options, the counter-based random stream and the sampler."""

from .params import SamplingParams
from .rng import uniform
from .sampler import PendingTokens, Sampler

__all__ = ["PendingTokens", "Sampler", "SamplingParams", "uniform"]
