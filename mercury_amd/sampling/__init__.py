"""Sampling: greedy, temperature, nucleus; per-request random streams."""

from .sampler import Sampler, uniform_for

__all__ = ["Sampler", "uniform_for"]
