"""Sampling parameters and the sampler over float32 logits."""

from .params import SamplingParams

__all__ = ["SamplingParams"]
