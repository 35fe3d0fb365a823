"""Sampling."""

from .sampler import GREEDY, Sampler, SamplingParams, uniform_for

__all__ = ["GREEDY", "Sampler", "SamplingParams", "uniform_for"]
