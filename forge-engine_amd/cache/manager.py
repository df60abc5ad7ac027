"""The cache manager: which pages and which state slot each request holds.

Host-side bookkeeping only (the device tensors belong to the model runner).
Layer calls with the same cache geometry form a group; each group has a pool of
pages of its own and, for each request, a block table of its own.  A request
also holds one state slot for fixed-size per-request state.

Life of a request: ``begin`` (slot leased, empty tables) -> ``reserve`` before
each step (pages for the tokens the step brings, all groups or none) ->
``commit`` after the step (length grows; pages that a window has passed go
back) -> ``end`` (everything goes back).  Nothing else frees pages.
"""

from __future__ import annotations

from dataclasses import dataclass, field

from .allocator import BlockAllocator, CacheCapacityError, StateSlotPool
from .spec import CacheNeeds

NO_PAGE = -1


@dataclass(frozen=True)
class CacheGroup:
    """Layer calls that share page geometry (and therefore tables)."""

    index: int
    kv_heads: int
    head_dim: int
    window: int | None
    slots: tuple[int, ...]  # cache slots (schedule indices that write) in this group
    value_dim: int = -1     # width of a value row (-1: head_dim; 0: the group holds keys only)

    @property
    def value_width(self) -> int:
        return self.head_dim if self.value_dim < 0 else self.value_dim


@dataclass
class RequestCache:
    request_id: str
    state_slot: int
    length: int = 0                                   # tokens whose keys are in the cache
    tables: list[list[int]] = field(default_factory=list)   # per group: page id per logical block, NO_PAGE if given back
    first_block: list[int] = field(default_factory=list)    # per group: logical blocks below this were given back
    lease: int = 0                                    # differs for every ``begin``: a request that ends and begins
                                                      # again under its old name holds other pages


def plan_groups(needs: list[CacheNeeds], schedule) -> tuple[list[CacheGroup], dict[int, tuple[int, int]]]:
    """Group the cache slots of a schedule by geometry.

    Returns the groups and a map cache slot -> (group index, index within the
    group's tensor)."""
    by_key: dict[tuple, list[int]] = {}
    for index, call in enumerate(schedule):
        paged = needs[index].paged
        if paged is None or call.cache != index:
            continue
        by_key.setdefault((paged.kv_heads, paged.head_dim, paged.window, paged.value_width), []).append(index)
    groups = []
    where: dict[int, tuple[int, int]] = {}
    for g, (key, slots) in enumerate(by_key.items()):
        groups.append(CacheGroup(g, key[0], key[1], key[2], tuple(slots), key[3]))
        for j, slot in enumerate(slots):
            where[slot] = (g, j)
    for index, call in enumerate(schedule):
        paged = needs[index].paged
        if paged is not None and call.cache != index:
            if call.cache not in where:
                raise ValueError(f"schedule entry {index} reads cache slot {call.cache}, which holds no pages")
            owner = needs[call.cache].paged
            if (owner.kv_heads, owner.head_dim, owner.value_width) != (paged.kv_heads, paged.head_dim, paged.value_width):
                raise ValueError(f"schedule entry {index} reads a cache of another geometry")
            # the owner's window decides which pages go back: a reader that looks further back
            # would read pages that are no longer the request's
            if owner.window is not None and (paged.window is None or paged.window > owner.window):
                raise ValueError(
                    f"schedule entry {index} looks back {paged.window or 'without limit'} but reads cache slot "
                    f"{call.cache}, which keeps only the last {owner.window} keys")
    return groups, where


class CacheManager:
    def __init__(self, groups: list[CacheGroup], *, block_size: int, block_capacity: int | list[int],
                 num_state_slots: int) -> None:
        if block_size < 1:
            raise ValueError("block_size must be at least 1")
        self.groups = list(groups)
        self.block_size = block_size
        capacities = block_capacity if isinstance(block_capacity, (list, tuple)) else [block_capacity] * len(groups)
        if len(capacities) != len(groups):
            raise ValueError("one page capacity per cache group is needed")
        self.pools = [BlockAllocator(c) for c in capacities]
        self.slots = StateSlotPool(num_state_slots)
        self._requests: dict[str, RequestCache] = {}
        self._leases = 0

    # ------------------------------------------------------------- queries
    def __contains__(self, request_id: str) -> bool:
        return request_id in self._requests

    def request(self, request_id: str) -> RequestCache:
        try:
            return self._requests[request_id]
        except KeyError:
            raise KeyError(f"unknown request '{request_id}'") from None

    def holds(self, entries: list[RequestCache]) -> bool:
        """Whether every record is still the live one of its request (none ended since)."""
        requests = self._requests
        return all(requests.get(entry.request_id) is entry for entry in entries)

    def live_requests(self) -> list[str]:
        return list(self._requests)

    def length(self, request_id: str) -> int:
        return self.request(request_id).length

    def blocks_for(self, tokens: int) -> int:
        return (tokens + self.block_size - 1) // self.block_size

    def pages_needed(self, request_id: str, new_length: int) -> list[int]:
        """Pages each group must still lease for the request to hold
        ``new_length`` tokens."""
        entry = self.request(request_id)
        want = self.blocks_for(new_length)
        return [max(0, want - len(table)) for table in entry.tables]

    def worst_case_pages(self, total_tokens: int, step_tokens: int | None = None) -> list[int]:
        """Upper bound, per group, of the pages a request of ``total_tokens`` ever holds at
        once.  A windowed group gives back the pages its window has passed after every step, so
        with at most ``step_tokens`` tokens of the request in a step it holds the window's keys
        and the step's, which touch one page more than their count fills; without
        ``step_tokens`` the bound is the whole length."""
        whole = self.blocks_for(total_tokens)
        bounds = []
        for group in self.groups:
            if group.window is None or step_tokens is None:
                bounds.append(whole)
            else:
                bounds.append(min(whole, self.blocks_for(group.window - 1 + step_tokens) + 1))
        return bounds

    @property
    def allocated_pages(self) -> int:
        return sum(pool.leased_count for pool in self.pools)

    # ------------------------------------------------------------ lifecycle
    def begin(self, request_id: str) -> RequestCache:
        if request_id in self._requests:
            raise ValueError(f"request '{request_id}' already holds cache")
        self._leases += 1
        entry = RequestCache(request_id, self.slots.lease(), 0,
                             [[] for _ in self.groups], [0 for _ in self.groups], self._leases)
        self._requests[request_id] = entry
        return entry

    def reserve(self, wanted: dict[str, int]) -> None:
        """Lease the pages that let each request grow to its new length.
        Either every request in ``wanted`` gets its pages in every group, or
        nothing changes and ``CacheCapacityError`` is raised."""
        plan: list[tuple[RequestCache, int, int]] = []
        totals = [0] * len(self.groups)
        for request_id, new_length in wanted.items():
            entry = self.request(request_id)
            if new_length < entry.length:
                raise ValueError(f"request '{request_id}' cannot shrink from {entry.length} to {new_length}")
            for g, count in enumerate(self.pages_needed(request_id, new_length)):
                if count:
                    plan.append((entry, g, count))
                    totals[g] += count
        for g, total in enumerate(totals):
            if total > self.pools[g].free_count:
                raise CacheCapacityError(
                    f"cache group {g} needs {total} pages but only {self.pools[g].free_count} are free")
        for entry, g, count in plan:
            entry.tables[g].extend(self.pools[g].allocate(count))

    def commit(self, request_id: str, new_length: int) -> None:
        """The step ran: the request now holds ``new_length`` tokens.  Pages
        that lie wholly before every window that a later token can look through
        go back to their pools."""
        entry = self.request(request_id)
        if new_length < entry.length or self.blocks_for(new_length) > min(
                (len(t) for t in entry.tables), default=self.blocks_for(new_length)):
            raise ValueError(f"request '{request_id}' has no pages for length {new_length}")
        entry.length = new_length
        for g, group in enumerate(self.groups):
            if group.window is None:
                continue
            # the next token sits at position new_length and reads keys > new_length - window
            first_needed = max(0, new_length - group.window + 1)
            keep_from = first_needed // self.block_size
            table = entry.tables[g]
            passed = [b for b in range(entry.first_block[g], min(keep_from, len(table)))]
            if passed:
                self.pools[g].release([table[b] for b in passed])
                for b in passed:
                    table[b] = NO_PAGE
                entry.first_block[g] = passed[-1] + 1

    def commit_single_tokens(self, entries: list[RequestCache]) -> None:
        """``commit`` for requests that each grew by one token (the decode step)."""
        windowed = any(group.window is not None for group in self.groups)
        for entry in entries:
            if windowed:
                self.commit(entry.request_id, entry.length + 1)
            else:
                if any(len(table) * self.block_size <= entry.length for table in entry.tables):
                    raise ValueError(f"request '{entry.request_id}' has no page for its next token")
                entry.length += 1

    def end(self, request_id: str) -> None:
        entry = self._requests.pop(request_id, None)
        if entry is None:
            raise KeyError(f"unknown request '{request_id}'")
        for g, table in enumerate(entry.tables):
            self.pools[g].release([page for page in table if page != NO_PAGE])
        self.slots.release([entry.state_slot])

    def check_invariants(self) -> None:
        """No page lost, held twice, or free and held at once."""
        for g, pool in enumerate(self.pools):
            held: list[int] = []
            for entry in self._requests.values():
                held.extend(page for page in entry.tables[g] if page != NO_PAGE)
            if len(held) != len(set(held)):
                raise AssertionError(f"group {g}: a page is held twice")
            if set(held) != set(pool.leased()):
                raise AssertionError(f"group {g}: leased pages and tables disagree")
            if pool.leased_count + pool.free_count != pool.capacity:
                raise AssertionError(f"group {g}: a page was lost")
        slots = [entry.state_slot for entry in self._requests.values()]
        if len(slots) != len(set(slots)) or set(slots) != set(self.slots.leased()):
            raise AssertionError("state slots and requests disagree")
