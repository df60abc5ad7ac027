"""The step function, the scheduler above it and the Python entry points."""

from .batch import StepBatch, StepEntry
from .loading import build_model, load_model, parse_dtype, random_model
from .runner import ModelRunner

__all__ = ["ModelRunner", "StepBatch", "StepEntry", "build_model", "load_model", "parse_dtype",
           "random_model"]
