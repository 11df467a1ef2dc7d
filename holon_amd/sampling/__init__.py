"""Sampling."""
from .sampler import Sampler, sequence_seed

__all__ = ["Sampler", "sequence_seed"]
