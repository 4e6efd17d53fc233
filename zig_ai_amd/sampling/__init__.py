"""Sampling: greedy, temperature, top-k, top-p, repetition penalty."""

from .sampler import SamplingParams, UniformStream, sample_rows, uniforms  # noqa: F401
