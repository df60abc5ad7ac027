"""The cache manager: deterministic page ids, all-or-nothing leases, windows
that give pages back, state slots, and no page lost, held twice or freed twice
under random orders of requests."""

from __future__ import annotations

import random

import pytest

from forge_engine_amd.cache import (NO_PAGE, BlockAllocator, CacheCapacityError, CacheGroup, CacheManager,
                                    CacheNeeds, FixedState, PagedKV, plan_groups)
from forge_engine_amd.parts import LayerCall


def manager(capacity=5, block_size=2, window=None, slots=4, groups=1):
    specs = [CacheGroup(g, 2, 16, window if g == 0 else None, (g,)) for g in range(groups)]
    return CacheManager(specs, block_size=block_size, block_capacity=capacity, num_state_slots=slots)


def grow(cache, request_id, new_length):
    cache.reserve({request_id: new_length})
    cache.commit(request_id, new_length)


def test_lowest_ids_first_and_holes_reused_in_release_order():
    # the tables the reference's tests pin (tests/test_cache.py:112,184 there)
    cache = manager(capacity=5, block_size=2)
    first, second = cache.begin("a"), cache.begin("b")
    grow(cache, "a", 3)
    grow(cache, "b", 3)
    assert first.tables[0] == [0, 1] and second.tables[0] == [2, 3]
    cache.end("a")
    grow(cache, "b", 4)
    assert second.tables[0] == [2, 3]             # the tail page is filled first
    grow(cache, "b", 5)
    assert second.tables[0] == [2, 3, 0]          # the hole released first comes back first
    assert cache.allocated_pages == 3
    cache.check_invariants()


def test_five_tokens_take_three_pages_of_two():
    cache = manager(capacity=4, block_size=2)
    entry = cache.begin("a")
    grow(cache, "a", 5)
    assert entry.tables[0] == [0, 1, 2] and entry.length == 5 and cache.allocated_pages == 3


def test_a_failed_lease_changes_nothing():
    cache = manager(capacity=3, block_size=2)
    cache.begin("a")
    cache.begin("b")
    grow(cache, "a", 2)
    with pytest.raises(CacheCapacityError, match="only 2 are free"):
        cache.reserve({"a": 4, "b": 4})      # needs 1 + 2 pages, 2 are free: neither request gets any
    assert cache.request("a").tables[0] == [0] and cache.request("b").tables[0] == []
    assert cache.allocated_pages == 1
    cache.reserve({"a": 4, "b": 2})
    cache.check_invariants()
    cache.end("a")
    cache.end("b")
    assert cache.allocated_pages == 0 and cache.slots.leased_count == 0


def test_double_release_and_unknown_requests_are_refused():
    pool = BlockAllocator(2)
    ids = pool.allocate(1)
    pool.release(ids)
    with pytest.raises(ValueError, match="not leased"):
        pool.release(ids)
    with pytest.raises(ValueError, match="twice"):
        pool.release([1, 1])
    cache = manager()
    cache.begin("a")
    with pytest.raises(ValueError, match="already"):
        cache.begin("a")
    cache.end("a")
    with pytest.raises(KeyError):
        cache.end("a")
    with pytest.raises(KeyError):
        cache.reserve({"zz": 3})


def test_commit_needs_reserved_pages_and_cannot_shrink():
    cache = manager()
    cache.begin("a")
    with pytest.raises(ValueError, match="no pages"):
        cache.commit("a", 3)
    grow(cache, "a", 3)
    with pytest.raises(ValueError, match="shrink"):
        cache.reserve({"a": 2})


def test_state_slots_are_leased_and_run_out():
    cache = manager(slots=2)
    assert cache.begin("a").state_slot == 0 and cache.begin("b").state_slot == 1
    with pytest.raises(CacheCapacityError, match="state slots"):
        cache.begin("c")
    assert "c" not in cache
    cache.end("a")
    assert cache.begin("c").state_slot == 0
    cache.check_invariants()


def test_window_gives_back_pages_it_has_passed():
    cache = manager(capacity=4, block_size=4, window=6)
    entry = cache.begin("a")
    grow(cache, "a", 9)       # next token at 9 reads keys 4..9: page 0 (keys 0..3) has been passed
    assert entry.tables[0] == [NO_PAGE, 1, 2] and cache.allocated_pages == 2
    grow(cache, "a", 13)      # next token at 13 reads keys 8..13: page 1 (keys 4..7) goes too
    assert entry.tables[0] == [NO_PAGE, NO_PAGE, 2, 0]
    for length in range(14, 60):    # a long request lives in a pool far smaller than its length
        grow(cache, "a", length)
        assert cache.allocated_pages <= 3
        first_needed = max(0, length - 6 + 1)
        assert all(page != NO_PAGE for page in entry.tables[0][first_needed // 4:])
        cache.check_invariants()
    cache.end("a")
    assert cache.allocated_pages == 0


def test_groups_have_pages_of_their_own_and_lease_together():
    cache = manager(capacity=3, block_size=4, window=4, groups=2)   # group 0 windowed, group 1 keeps all
    entry = cache.begin("a")
    grow(cache, "a", 12)
    assert entry.tables[1] == [0, 1, 2] and entry.tables[0] == [NO_PAGE, NO_PAGE, 2]
    with pytest.raises(CacheCapacityError, match="group 1"):
        cache.reserve({"a": 13})         # the full group is exhausted; the windowed group must not lease either
    assert entry.tables[0] == [NO_PAGE, NO_PAGE, 2]
    cache.check_invariants()


def test_plan_groups_by_geometry_and_shared_slots():
    needs = [CacheNeeds(PagedKV(2, 16)), CacheNeeds(PagedKV(2, 16, window=8)), CacheNeeds(PagedKV(2, 16)),
             CacheNeeds(state=FixedState((4,))), CacheNeeds(PagedKV(2, 16))]
    schedule = [LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(2, 3), LayerCall(1, 0, writes_cache=False)]
    groups, where = plan_groups(needs, schedule)
    assert [(g.window, g.slots) for g in groups] == [(None, (0, 2)), (8, (1,))]
    assert where == {0: (0, 0), 2: (0, 1), 1: (1, 0)}
    with pytest.raises(ValueError, match="holds no pages"):
        plan_groups([CacheNeeds(state=FixedState((4,))), CacheNeeds(PagedKV(2, 16))],
                    [LayerCall(0, 0), LayerCall(1, 0, writes_cache=False)])


def test_a_reader_may_not_look_further_back_than_the_cache_it_reads_keeps():
    # the owner's window decides which pages go back; a reader without a window, or with a wider one,
    # would read pages that are no longer the request's
    owner = CacheNeeds(PagedKV(2, 16, window=8))
    for reader_window in (None, 9):
        with pytest.raises(ValueError, match="keeps only the last 8 keys"):
            plan_groups([owner, CacheNeeds(PagedKV(2, 16, window=reader_window))],
                        [LayerCall(0, 0), LayerCall(1, 0, writes_cache=False)])
    for reader_window in (8, 3):
        plan_groups([owner, CacheNeeds(PagedKV(2, 16, window=reader_window))],
                    [LayerCall(0, 0), LayerCall(1, 0, writes_cache=False)])
    # an owner that keeps everything serves any reader
    plan_groups([CacheNeeds(PagedKV(2, 16)), CacheNeeds(PagedKV(2, 16, window=5))],
                [LayerCall(0, 0), LayerCall(1, 0, writes_cache=False)])


def test_worst_case_of_a_windowed_group_is_its_window_and_a_step():
    cache = manager(capacity=64, block_size=4, window=6, groups=2)      # group 0 windowed, group 1 keeps all
    assert cache.worst_case_pages(100) == [25, 25]
    assert cache.worst_case_pages(100, step_tokens=1) == [3, 25]        # 6 keys touch at most 3 pages of 4
    assert cache.worst_case_pages(100, step_tokens=8) == [5, 25]
    assert cache.worst_case_pages(5, step_tokens=8) == [2, 2]
    # the bound holds: decode a long request one token at a time, and in steps of eight
    for step in (1, 8):
        entry = cache.begin(f"r{step}")
        for length in range(step, 100, step):
            cache.reserve({entry.request_id: length})
            assert sum(page != NO_PAGE for page in entry.tables[0]) <= cache.worst_case_pages(100, step_tokens=step)[0]
            cache.commit(entry.request_id, length)
        cache.end(entry.request_id)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted(seed):
    rng = random.Random(seed)
    cache = manager(capacity=24, block_size=4, window=rng.choice([None, 5, 16]), slots=5, groups=2)
    live: dict[str, int] = {}
    counter = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(live) < 5:
            counter += 1
            name = f"r{counter}"
            cache.begin(name)
            live[name] = 0
        elif action < 0.85 and live:
            chosen = rng.sample(sorted(live), rng.randint(1, len(live)))
            wanted = {name: live[name] + rng.choice([1, 1, 1, 2, 7, 13]) for name in chosen}
            before = {name: [list(t) for t in cache.request(name).tables] for name in live}
            try:
                cache.reserve(wanted)
            except CacheCapacityError:
                after = {name: [list(t) for t in cache.request(name).tables] for name in live}
                assert after == before
                victim = max(live, key=live.get)
                cache.end(victim)
                del live[victim]
            else:
                for name, length in wanted.items():
                    cache.commit(name, length)
                    live[name] = length
        elif live:
            name = rng.choice(sorted(live))
            cache.end(name)
            del live[name]
        cache.check_invariants()
    for name in list(live):
        cache.end(name)
    assert cache.allocated_pages == 0 and cache.slots.leased_count == 0
    assert all(pool.free_count == pool.capacity for pool in cache.pools)
