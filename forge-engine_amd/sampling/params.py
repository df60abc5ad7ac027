"""Parameters of token sampling; names, defaults and checks follow the
reference (src/forge_engine/sampling.py:14-46)."""

from __future__ import annotations

import math
from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    temperature: float = 0.0
    top_k: int | None = None
    top_p: float = 1.0
    min_p: float = 0.0
    max_new_tokens: int = 256
    stop_strings: tuple[str, ...] = ()
    seed: int | None = None

    def __post_init__(self) -> None:
        if not math.isfinite(self.temperature) or self.temperature < 0.0:
            raise ValueError("temperature must be finite and non-negative")
        if self.top_k is not None and self.top_k < 1:
            raise ValueError("top_k must be at least 1")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0, 1]")
        if not 0.0 <= self.min_p <= 1.0:
            raise ValueError("min_p must be in [0, 1]")
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        if any(not stop for stop in self.stop_strings):
            raise ValueError("stop strings must be non-empty")
        if len(set(self.stop_strings)) != len(self.stop_strings):
            raise ValueError("stop strings must be unique")

    @property
    def greedy(self) -> bool:
        return self.temperature == 0.0


def normalize_stop_strings(values) -> tuple[str, ...]:
    """Optional command-line list of stop strings to a tuple."""
    return () if values is None else tuple(values)
