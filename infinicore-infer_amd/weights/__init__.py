"""Weights: loading from safetensors by name, random-weights model folders."""
from .loader import IGNORED_PATTERNS, WeightError, WeightSpec, load_weights
from .random_init import init_random_weights, random_state_dict, standard_normal, write_random_model

__all__ = ["IGNORED_PATTERNS", "WeightError", "WeightSpec", "load_weights", "init_random_weights", "random_state_dict", "standard_normal",
           "write_random_model"]
