"""What a mixer asks of the cache manager, and what it is handed in a step."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping


@dataclass(frozen=True)
class PagedKV:
    """Keys and values in pages.  ``window`` None: every key is kept; else only
    the last ``window`` keys of a request are ever read again, and pages that
    the window has passed go back to the pool."""

    kv_heads: int
    head_dim: int
    window: int | None = None
    value_dim: int | None = None   # width of a value row: None, as wide as a key; 0: keys only, no value pages at all

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class FixedState:
    """Per-request state of fixed size (one slot per live request)."""

    shape: tuple[int, ...]
    dtype: Any = None  # a torch dtype; None: float32


@dataclass(frozen=True)
class CacheNeeds:
    """``state``: one ``FixedState``, or several by name, each with a shape and a dtype of its own
    (a recurrent state in float32 beside the tail of a short convolution in bfloat16, say)."""

    paged: PagedKV | None = None
    state: FixedState | Mapping[str, FixedState] | None = None

    def states(self) -> dict[str, FixedState]:
        """The states by name; a single unnamed one is called ``state``."""
        if self.state is None:
            return {}
        if isinstance(self.state, FixedState):
            return {"state": self.state}
        return dict(self.state)


@dataclass
class CacheView:
    """What one layer call sees of the cache in one step.

    ``key_pages`` [blocks, kv_heads, block_size, head_dim] and ``value_pages``
    (transposed) [blocks, kv_heads, value width, block_size] of this call's cache slot (None for a
    mixer that keeps keys only); ``block_table``: int32 [sequences, max_blocks] of the
    slot's group (entry -1: no page); ``states``: by name, [slots, *shape] of each of this call's
    fixed-size states, indexed by ``StepBatch.state_slots``; ``state``: the only one, for a mixer
    that has one.
    """

    key_pages: Any = None
    value_pages: Any = None
    block_table: Any = None
    block_size: int = 0
    window: int | None = None
    states: dict = field(default_factory=dict)

    @property
    def state(self) -> Any:
        if len(self.states) != 1:
            raise AttributeError(f"this call has {len(self.states)} fixed-size states: name one in ``states``")
        return next(iter(self.states.values()))
