"""Sampling parameters and the sampler over float32 logits."""

from .params import SamplingParams, normalize_stop_strings

__all__ = ["SamplingParams", "normalize_stop_strings"]
