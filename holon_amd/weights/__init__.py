"""Weights: the safetensors loader and the random-weights mode."""
from .loader import WeightError, load_weights, map_name, unmap_name
from .random_init import fill_random, random_tensor, write_random_model

__all__ = ["WeightError", "load_weights", "map_name", "unmap_name", "fill_random", "random_tensor",
           "write_random_model"]
