"""Engine-side configuration: sampling defaults and scheduler limits.

Names and defaults follow the reference: ``EngineConfig``
(src/forge_engine/config.py:11-37) and ``SchedulerConfig``
(scheduler.py:56-76).  ``prefill_chunk``, ``admission``, ``max_context`` and
``num_state_slots`` are additions for portions of prompts, the choice of what
happens when pages run out, and per-request state slots.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..sampling.params import SamplingParams


@dataclass(frozen=True)
class EngineConfig:
    max_new_tokens: int = 256
    temperature: float = 0.0
    top_k: int | None = None
    top_p: float = 1.0
    min_p: float = 0.0
    stop_strings: tuple[str, ...] = ()
    seed: int | None = None

    def __post_init__(self) -> None:
        self.sampling_params()

    def sampling_params(self) -> SamplingParams:
        return SamplingParams(
            temperature=self.temperature, top_k=self.top_k, top_p=self.top_p, min_p=self.min_p,
            max_new_tokens=self.max_new_tokens, stop_strings=self.stop_strings, seed=self.seed)


@dataclass(frozen=True)
class SchedulerConfig:
    max_requests: int = 16
    max_batch_size: int = 8
    token_budget: int = 256
    block_size: int = 16
    block_capacity: int | tuple[int, ...] = 1024   # pages of every cache group's pool, or one count per group
    prefill_chunk: int | None = None      # longest portion of one prompt in a step (None: the budget)
    admission: str = "reserve"            # "reserve": worst-case pages at submit; "preempt": on demand
    max_context: int | None = None        # longest prompt + new tokens accepted (None: the pool's size)
    num_state_slots: int | None = None    # per-request state slots (None: max_requests)
    overlap_decode: bool = True           # steady greedy decode steps take their tokens on the device; the host reads a step late

    def capacities(self, groups: int) -> list[int]:
        """The page capacity of each of ``groups`` cache groups."""
        if isinstance(self.block_capacity, tuple):
            if len(self.block_capacity) != groups:
                raise ValueError(f"block_capacity names {len(self.block_capacity)} cache groups, the model has {groups}")
            return list(self.block_capacity)
        return [self.block_capacity] * groups

    def __post_init__(self) -> None:
        for name in ("max_requests", "max_batch_size", "token_budget", "block_size"):
            if getattr(self, name) < 1:
                raise ValueError(f"{name} must be at least 1")
        if isinstance(self.block_capacity, (list, tuple)):
            object.__setattr__(self, "block_capacity", tuple(int(c) for c in self.block_capacity))
        capacities = self.block_capacity if isinstance(self.block_capacity, tuple) else (self.block_capacity,)
        if not capacities or min(capacities) < 1:
            raise ValueError("block_capacity must be at least 1")
        if self.prefill_chunk is not None and self.prefill_chunk < 1:
            raise ValueError("prefill_chunk must be at least 1")
        if self.admission not in ("reserve", "preempt"):
            raise ValueError("admission must be 'reserve' or 'preempt'")
        if self.max_context is not None and self.max_context < 1:
            raise ValueError("max_context must be at least 1")
        if self.num_state_slots is not None and self.num_state_slots < 1:
            raise ValueError("num_state_slots must be at least 1")
