"""Sampling parameters and the GPU sampler."""

from tokamak_amd.sampling.params import SamplingParams

__all__ = ["SamplingParams"]
