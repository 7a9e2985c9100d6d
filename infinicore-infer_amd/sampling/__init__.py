"""Sampling: parameters, reproducible uniform draws, the device sampler's rules."""
from .params import SamplingParams, uniform_draw

__all__ = ["SamplingParams", "uniform_draw"]
