"""Sampling parameters and the GPU sampler."""

from .params import SamplingParams

__all__ = ["SamplingParams"]
