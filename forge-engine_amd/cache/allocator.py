"""Fixed pools of page ids and of state slots.

The order in which ids are handed out is deterministic, as in the reference's
pool (src/forge_engine/cache.py:145-244): the lowest free id is leased first,
and among released ids the one released first is leased first (its tests pin
the tables (0, 1, 2) and, after a release, (2, 3, 0): tests/test_cache.py:112,184).
Leasing is all-or-nothing; releasing an id that is not leased, or twice, raises
before anything changes.
"""

from __future__ import annotations


class CacheCapacityError(RuntimeError):
    """The pool cannot supply the pages or slots asked for."""


class BlockAllocator:
    def __init__(self, capacity: int) -> None:
        if capacity < 1:
            raise ValueError("capacity must be at least 1")
        self._capacity = capacity
        self._free = list(range(capacity - 1, -1, -1))  # a stack: the next lease is at the end
        self._leased: set[int] = set()

    @property
    def capacity(self) -> int:
        return self._capacity

    @property
    def free_count(self) -> int:
        return len(self._free)

    @property
    def leased_count(self) -> int:
        return len(self._leased)

    def leased(self) -> frozenset[int]:
        return frozenset(self._leased)

    def allocate(self, count: int) -> list[int]:
        if count < 0:
            raise ValueError("cannot lease a negative number of pages")
        if count == 0:
            return []
        if count > len(self._free):
            raise CacheCapacityError(
                f"the pool needs {count} pages but only {len(self._free)} are free")
        taken = self._free[-count:][::-1]
        del self._free[-count:]
        self._leased.update(taken)
        return taken

    def release(self, ids) -> None:
        ids = list(ids)
        if len(set(ids)) != len(ids):
            raise ValueError("cannot release a page twice in one call")
        unknown = [i for i in ids if i not in self._leased]
        if unknown:
            raise ValueError(f"cannot release pages that are not leased: {unknown}")
        self._leased.difference_update(ids)
        self._free.extend(reversed(ids))


class StateSlotPool(BlockAllocator):
    """Slots of fixed-size per-request state: one id per live request."""

    def lease(self) -> int:
        try:
            return self.allocate(1)[0]
        except CacheCapacityError:
            raise CacheCapacityError(f"all {self.capacity} state slots are in use") from None
