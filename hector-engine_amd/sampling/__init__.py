"""Greedy, temperature, top-k, top-p and penalty sampling."""
from .rng import uniform_u32
from .sampler import Sampler, SamplingConfig, window_counts
