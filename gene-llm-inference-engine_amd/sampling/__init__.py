"""Greedy, temperature, top-k and top-p sampling with the reference's random generator."""
from .sampler import Sampler, SamplerConfig, UniformStream, filtered_draw, sample_rows, sample_rows_on_device
