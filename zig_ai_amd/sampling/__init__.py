"""Sampling: greedy, temperature, top-k, top-p, repetition penalty."""

from .sampler import SamplingParams, UniformStream, sample_rows  # noqa: F401
