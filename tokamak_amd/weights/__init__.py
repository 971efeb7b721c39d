"""Weights: sources (safetensors folder, seeded random), validation, binding."""

from tokamak_amd.weights.loader import WeightError, load_weights, validate
from tokamak_amd.weights.random_init import write_random_model
from tokamak_amd.weights.sources import RandomSource, SafetensorsSource
from tokamak_amd.weights.spec import TensorSpec

__all__ = [
    "RandomSource",
    "SafetensorsSource",
    "TensorSpec",
    "WeightError",
    "load_weights",
    "validate",
    "write_random_model",
]
