"""Weights: loading safetensors by tensor name, and seeded random models."""

from .loader import WeightsError, checkpoint_files, load_weights, storage_dtype
from .random_init import fill_random_weights, random_tensors, write_random_model

__all__ = ["WeightsError", "checkpoint_files", "fill_random_weights", "load_weights", "random_tensors",
           "storage_dtype", "write_random_model"]
