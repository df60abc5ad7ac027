"""What a mixer asks of the cache manager, and what it is handed in a step."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any


@dataclass(frozen=True)
class PagedKV:
    """Keys and values in pages.  ``window`` None: every key is kept; else only
    the last ``window`` keys of a request are ever read again, and pages that
    the window has passed go back to the pool."""

    kv_heads: int
    head_dim: int
    window: int | None = None


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (one slot per live request)."""

    shape: tuple[int, ...]
    dtype: Any = None  # a torch dtype; None: float32


@dataclass(frozen=True)
class CacheNeeds:
    paged: PagedKV | None = None
    state: FixedState | None = None


@dataclass
class CacheView:
    """What one layer call sees of the cache in one step.

    ``key_pages`` [blocks, kv_heads, block_size, head_dim] and ``value_pages``
    (transposed) [blocks, kv_heads, head_dim, block_size] of this call's cache slot; ``block_table``: int32 [sequences, max_blocks] of the
    slot's group (entry -1: no page); ``state``: [slots, *shape] of this call's
    fixed-size state, indexed by ``StepBatch.state_slots``.
    """

    key_pages: Any = None
    value_pages: Any = None
    block_table: Any = None
    block_size: int = 0
    window: int | None = None
    state: Any = None
