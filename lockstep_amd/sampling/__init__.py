"""Sampling: counter-based uniform draws, greedy and nucleus sampling."""

from .philox import philox_4x32, uid_key, uniform
from .sampler import Sampler, greedy, top_p

__all__ = ["philox_4x32", "uid_key", "uniform", "Sampler", "greedy", "top_p"]
