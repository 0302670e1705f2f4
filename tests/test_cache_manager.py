"""The cache manager: lowest page first and immediate reuse, all-or-nothing reservations, windows
that give pages back, state slots, and no page lost, held twice or freed twice under random orders."""
import random

import pytest

import vipera_rs_amd  # noqa: F401
from vipera_rs_amd.cache import (RESERVE_NEVER_FITS, RESERVE_NO_PAGES, RESERVE_NO_SLOT, RESERVE_OK, CacheGroupSpec,
                                 CacheManager)
from vipera_rs_amd.errors import InfeasibleError, InvalidArgumentError


def test_lowest_page_first_and_released_pages_are_reused_at_once():
    cache = CacheManager([CacheGroupSpec(4, 8)], 4)
    cache.reserve(1, 0, 9)                      # three pages (crates/vipera-runtime/src/kv.rs:590-598)
    assert cache.table(1, 0) == [0, 1, 2]
    cache.reserve(2, 0, 4)
    assert cache.table(2, 0) == [3]
    cache.release(1)
    cache.reserve(3, 0, 8)
    assert cache.table(3, 0) == [0, 1]          # the pages just given back, lowest first
    assert cache.check() == ""


def test_growing_a_request_keeps_its_pages():
    cache = CacheManager([CacheGroupSpec(16, 4)], 2)
    cache.reserve(7, 0, 10)
    first = cache.table(7, 0)
    cache.reserve(7, 10, 17)
    assert cache.table(7, 0)[:1] == first and len(cache.table(7, 0)) == 2
    cache.reserve(7, 17, 18)
    assert len(cache.table(7, 0)) == 2 and cache.used_blocks(0) == 2


def test_a_failed_reservation_changes_nothing():
    cache = CacheManager([CacheGroupSpec(4, 4), CacheGroupSpec(4, 2, window=6)], 2)
    cache.reserve(1, 0, 8)                      # 2 pages in each group
    before = (cache.free_blocks(0), cache.free_blocks(1), cache.free_slots())
    assert cache.try_reserve(2, 0, 8) == RESERVE_NO_PAGES       # the second group has none left
    assert (cache.free_blocks(0), cache.free_blocks(1), cache.free_slots()) == before
    assert not cache.knows(2) and cache.table(2, 0) == []
    assert cache.try_reserve(1, 8, 40) == RESERVE_NEVER_FITS    # more than the first pool holds in total
    assert cache.table(1, 0) == [0, 1] and cache.check() == ""
    with pytest.raises(InfeasibleError, match="cache is full"):
        cache.reserve(2, 0, 8)
    with pytest.raises(InfeasibleError, match="more pages"):
        cache.reserve(1, 8, 40)


def test_slots_run_out_and_come_back():
    cache = CacheManager([CacheGroupSpec(4, 16)], 2)
    cache.reserve(1, 0, 1)
    cache.reserve(2, 0, 1)
    assert sorted([cache.slot(1), cache.slot(2)]) == [0, 1]
    assert cache.try_reserve(3, 0, 1) == RESERVE_NO_SLOT and cache.used_blocks(0) == 2
    cache.release(1)
    assert cache.try_reserve(3, 0, 1) == RESERVE_OK and cache.slot(3) in (0, 1) and cache.slot(1) == -1
    with pytest.raises(InvalidArgumentError):
        cache.release(99)


def test_a_window_gives_pages_back_behind_it():
    cache = CacheManager([CacheGroupSpec(4, 16, window=6)], 2)
    cache.reserve(1, 0, 10)
    assert cache.table(1, 0) == [0, 1, 2]
    cache.advance(1, 10)          # the next token is at 10 and sees 5..10: page 0 (positions 0..3) is free again
    assert cache.table(1, 0) == [-1, 1, 2] and cache.free_blocks(0) == 14
    cache.reserve(1, 10, 11)      # position 10 lies in page 2: nothing new
    assert cache.table(1, 0) == [-1, 1, 2]
    cache.advance(1, 13)          # sees 8..13
    assert cache.table(1, 0) == [-1, -1, 2]
    cache.reserve(1, 13, 14)
    assert cache.table(1, 0) == [-1, -1, 2, 1] or cache.table(1, 0)[3] in (0, 1)   # a freed page is used again
    # a portion holds its whole window: positions 20+1-6 .. 29
    cache.advance(1, 20)
    cache.reserve(1, 20, 30)
    table = cache.table(1, 0)
    assert all(p >= 0 for p in table[15 // 4:8]) and all(p < 0 for p in table[:15 // 4])
    assert cache.check() == ""
    assert cache.blocks_needed(0, 1000, 1) <= 3 and cache.blocks_needed(0, 1000, 16) >= (6 - 1 + 16) // 4


def test_groups_have_pools_of_their_own():
    cache = CacheManager([CacheGroupSpec(8, 10), CacheGroupSpec(8, 3, window=8)], 4)
    for step in range(1, 60):
        cache.reserve(1, step - 1, step)
        cache.advance(1, step)
    assert cache.used_blocks(0) == 8 and cache.used_blocks(1) <= 2
    cache.release(1)
    assert cache.used_blocks(0) == 0 and cache.used_blocks(1) == 0 and cache.check() == ""


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_no_page_and_hold_none_twice(seed):
    rng = random.Random(seed)
    groups = [CacheGroupSpec(rng.choice([4, 8, 16]), rng.randrange(8, 40)),
              CacheGroupSpec(rng.choice([4, 8]), rng.randrange(6, 20), window=rng.randrange(5, 40))]
    cache = CacheManager(groups, 5)
    lengths = {}
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(lengths) < 7:
            total = rng.randrange(1, 50)
            if cache.try_reserve(next_id, 0, total) == RESERVE_OK:
                lengths[next_id] = total
                cache.advance(next_id, total)
            next_id += 1
        elif action < 0.75 and lengths:
            rid = rng.choice(list(lengths))
            grow = rng.randrange(1, 20)
            if cache.try_reserve(rid, lengths[rid], lengths[rid] + grow) == RESERVE_OK:
                lengths[rid] += grow
                cache.advance(rid, lengths[rid])
        elif lengths:
            rid = rng.choice(list(lengths))
            cache.release(rid)
            del lengths[rid]
        problem = cache.check()
        assert problem == "", problem
        held = set()
        for rid in lengths:
            for g in range(2):
                for page in cache.table(rid, g):
                    if page >= 0:
                        assert (g, page) not in held, f"page {page} of group {g} is held twice"
                        held.add((g, page))
        for g in range(2):
            assert cache.used_blocks(g) == sum(1 for gg, _ in held if gg == g)
            assert cache.used_blocks(g) + cache.free_blocks(g) == groups[g].num_blocks
        assert cache.live_requests() == len(lengths) and cache.free_slots() == 5 - len(lengths)
    for rid in list(lengths):
        cache.release(rid)
    assert all(cache.free_blocks(g) == groups[g].num_blocks for g in range(2)) and cache.check() == ""


def test_bad_geometry_is_refused():
    with pytest.raises(InvalidArgumentError):
        CacheManager([CacheGroupSpec(0, 4)], 1)
    with pytest.raises(InvalidArgumentError):
        CacheManager([CacheGroupSpec(4, 4)], 0)


def test_cache_groups_may_differ_in_page_size_and_pool_size():
    """One number for every group, or one per group in the order in which the run order first needs each; a page
    size that a mixer asks for itself stands; the engine's list has to match the number of groups."""
    from vipera_rs_amd.cache import group_keys, group_position_bytes, plan_groups
    from vipera_rs_amd.errors import InvalidArgumentError
    from vipera_rs_amd.models import CacheNeed
    from vipera_rs_amd.parts import KVCacheSpec, StateSpec
    needs = [CacheNeed(0, KVCacheSpec(2, 16, 0), None), CacheNeed(1, KVCacheSpec(2, 16, 21), None),
             CacheNeed(2, None, StateSpec((4,))), CacheNeed(3, KVCacheSpec(1, 32, 0, block_size=64), None),
             CacheNeed(1, KVCacheSpec(2, 16, 21), None), CacheNeed(5, KVCacheSpec(4, 8, 0), None)]
    assert group_keys(needs) == [(0, 0), (21, 0), (0, 64)]
    same = plan_groups(needs, 16, 10)
    assert [(g.block_size, g.num_blocks, g.window) for g in same] == [(16, 10, 0), (16, 10, 21), (64, 10, 0)]
    each = plan_groups(needs, [16, 8, 32], [10, 40, 3])
    assert [(g.block_size, g.num_blocks, g.window) for g in each] == [(16, 10, 0), (8, 40, 21), (64, 3, 0)]
    with pytest.raises(InvalidArgumentError, match="2 values for 3 cache groups"):
        plan_groups(needs, 16, [10, 40])
    # bytes per cached position and group: owners only (entry 4 reads entry 1's cache)
    assert group_position_bytes(needs, 2) == [(2 * 32 + 4 * 16) * 2, 2 * 32 * 2, 1 * 64 * 2]
    cache = CacheManager(each, 2)
    assert cache.reserve(7, 0, 100) is None
    assert [cache.used_blocks(g) for g in range(3)] == [7, 13, 2] and cache.check() == ""
    cache.advance(7, 100)                     # position 100 will see 80..100: pages 10, 11, 12 of 8 positions stay
    assert [cache.used_blocks(g) for g in range(3)] == [7, 3, 2]
    assert cache.allocate_micros() >= 0
