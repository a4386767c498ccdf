"""The cache manager on the CPU: pages, block tables, groups, windows, request slots.

The allocator's cases follow the reference's slot allocator (app/server.cpp:96-128: acquire until
empty, release refuses what is not in use) and its cache tests (tests/unit_tests.cpp:173-196:
out-of-range and budget errors), at page granularity."""
import random

import pytest
import torch

from tlie_amd import EngineError, ErrorCode
from tlie_amd.cache import ABSENT, CacheManager, PageAllocator, RunNeed
from tlie_amd.parts import CacheNeed, StateNeed


def test_allocator_fifo_all_or_nothing_and_double_free():
    pool = PageAllocator(4)
    assert pool.alloc(3) == [0, 1, 2] and pool.num_free == 1
    assert pool.alloc(2) is None and pool.num_free == 1          # nothing taken
    pool.release([1])
    assert pool.alloc(2) == [3, 1]                                # FIFO: the returned page comes last
    with pytest.raises(EngineError):
        pool.release([7])
    pool.release([0])
    with pytest.raises(EngineError):
        pool.release([0])                                         # freed twice
    with pytest.raises(EngineError):
        pool.release([2, 2])
    assert pool.in_use(2) and pool.num_used == 3                  # a refused call frees nothing
    with pytest.raises(EngineError):
        PageAllocator(0)


def manager(num_pages=8, page_size=4, max_requests=3, window=None, state=False, runs=2):
    needs = [RunNeed(cache_of=i, cache=CacheNeed((2, 2), 8, window), state=StateNeed((5,)) if state else None) for i in range(runs)]
    return CacheManager(needs, page_size, num_pages, max_requests, torch.float32, "cpu", max_positions=64)


def test_pages_follow_length_and_come_back():
    cache = manager()
    assert cache.admit("a") == 0 and cache.admit("b") == 1
    assert cache.pages_needed("a", 5) == [2]
    cache.reserve("a", 5)
    assert cache.page_list("a", 0) == [0, 1] and cache.length("a") == 0
    assert cache.rows("a", 0, 3, 2) == [3, 4]                     # position 3 on page 0, position 4 on page 1 row 0
    cache.commit("a", 5)
    assert cache.length("a") == 5 and cache.pages_needed("a", 3) == [0] and cache.pages_needed("a", 4) == [1]
    cache.reserve("b", 9)
    cache.commit("b", 9)
    assert cache.page_list("b", 0) == [2, 3, 4] and cache.free_pages() == [3]
    assert cache.can_reserve([("a", 3), ("b", 8)]) and not cache.can_reserve([("a", 4), ("b", 12)])
    with pytest.raises(EngineError) as caught:
        cache.reserve("b", 16)
    assert caught.value.code == ErrorCode.OUT_OF_MEMORY and cache.page_list("b", 0) == [2, 3, 4]
    cache.release("a")
    cache.check()
    assert cache.free_pages() == [5]
    cache.admit("c")                                              # the slot of "a" is used again
    assert cache.slot("c") == 0
    cache.reserve("c", 16)
    assert cache.page_list("c", 0) == [5, 6, 7, 0]                # FIFO: the pages "a" gave back come last
    cache.check()
    with pytest.raises(EngineError):
        cache.commit("c", 17)                                     # more than was reserved
    with pytest.raises(EngineError):
        cache.admit("c")
    with pytest.raises(EngineError):
        cache.length("nobody")
    with pytest.raises(EngineError) as caught:
        cache.reserve("c", 65)
    assert caught.value.code == ErrorCode.OUT_OF_BOUNDS           # past the model's positions


def test_a_step_reserves_for_all_its_requests_or_for_none():
    cache = manager()                                             # 8 pages of 4 positions
    for name in "abc":
        cache.admit(name)
    assert cache.reserve_all([("a", 5), ("b", 9)])                # 2 + 3 pages
    assert cache.page_list("a", 0) == [0, 1] and cache.page_list("b", 0) == [2, 3, 4]
    cache.commit("a", 5)
    cache.commit("b", 9)
    before = cache.held("a").serial, cache.held("b").serial
    assert not cache.reserve_all([("a", 3), ("c", 9), ("b", 4)])  # 0 + 3 + 1 pages, 3 are free
    assert cache.page_list("a", 0) == [0, 1] and cache.page_list("c", 0) == [] and cache.free_pages() == [3]
    assert cache.reserve_all([("a", 3), ("c", 8), ("b", 4)])      # 0 + 2 + 1
    assert cache.page_list("c", 0) == [5, 6] and cache.page_list("b", 0) == [2, 3, 4, 7]
    with pytest.raises(EngineError) as caught:
        cache.reserve_all([("a", 60)])
    assert caught.value.code == ErrorCode.OUT_OF_BOUNDS
    with pytest.raises(EngineError):
        cache.reserve_all([("a", 0)])
    cache.check()
    # an admission's serial tells a request's name from its next use
    cache.release("a")
    cache.admit("a")
    assert cache.held("a").serial not in before and cache.held("b").serial == before[1]


def test_a_step_that_did_not_run_gives_its_reservation_back():
    """What a step reserved and then did not run (its launch raised) goes back; the request keeps
    the pages its committed positions lie on, and the next reservation may get other pages."""
    cache = manager()                                             # 8 pages of 4 positions
    cache.admit("a")
    cache.admit("b")
    assert cache.reserve_all([("a", 6)])
    cache.commit("a", 6)                                          # pages 0, 1
    assert cache.reserve_all([("a", 9), ("b", 3)])                # "a" up to 15 positions: pages 2, 3; "b": page 4
    assert cache.page_list("a", 0) == [0, 1, 2, 3] and cache.free_pages() == [3]
    cache.unreserve("a")
    cache.unreserve("b")
    assert cache.page_list("a", 0) == [0, 1] and cache.page_list("b", 0) == [] and cache.free_pages() == [6]
    assert cache.length("a") == 6
    cache.check()
    cache.unreserve("a")                                          # nothing spare: nothing happens
    assert cache.page_list("a", 0) == [0, 1]
    assert cache.reserve_all([("b", 3), ("a", 2)])                # 1 + 0: the freed pages come back in the order of their release
    cache.commit("a", 2)
    assert cache.reserve_all([("a", 1)])
    assert cache.page_list("a", 0)[:2] == [0, 1] and len(cache.page_list("a", 0)) == 3
    cache.check()
    with pytest.raises(EngineError):
        cache.unreserve("nobody")


def test_request_slots_run_out_and_state_starts_at_zero():
    cache = manager(max_requests=2, state=True)
    assert len(cache.state_areas) == 2 and cache.state_areas[0].shape == (2, 5)
    cache.admit("a")
    cache.admit("b")
    with pytest.raises(EngineError) as caught:
        cache.admit("c")
    assert caught.value.code == ErrorCode.OUT_OF_MEMORY
    cache.bindings[0].state[cache.slot("b")] += 3.0
    cache.release("b")
    assert cache.admit("c") == 1 and float(cache.bindings[0].state[1].abs().sum()) == 0.0
    assert cache.bindings[0].state is not cache.bindings[1].state


def test_pages_of_other_shapes_and_types():
    """What a page looks like is the mixer's need, not the manager's: one vector per position in
    a type of its own, three planes, or attention's two planes per head, side by side; runs with
    the same window share page numbers whatever their pages hold."""
    needs = [RunNeed(0, CacheNeed((), 24, None, torch.float16)), RunNeed(1, CacheNeed((3,), 5, None)),
             RunNeed(2, CacheNeed((2, 2), 8, None)), RunNeed(0, CacheNeed((), 24, None, torch.float16))]
    cache = CacheManager(needs, 4, 6, 2, torch.float32, "cpu")
    assert len(cache.groups) == 1 and [b.group for b in cache.bindings] == [0, 0, 0, 0]
    assert cache.bindings[0].cache.shape == (6, 4 * 24) and cache.bindings[0].cache.dtype == torch.float16
    assert cache.bindings[1].cache.shape == (6, 3, 4 * 5) and cache.bindings[1].cache.dtype == torch.float32
    assert cache.bindings[2].cache.shape == (6, 2, 2, 4 * 8)
    assert cache.bindings[3].cache is cache.bindings[0].cache and not cache.bindings[3].writes
    assert CacheManager.page_bytes(needs, 4, torch.float32) == 4 * (24 * 2 + 15 * 4 + 32 * 4)
    assert CacheNeed((2, 3), 7).page_shape(16) == (2, 3, 112) and CacheNeed((), 9).values_per_position() == 9
    with pytest.raises(EngineError):         # a reader whose pages are of another type than the owner's
        CacheManager([RunNeed(0, CacheNeed((), 24, None, torch.float16)), RunNeed(0, CacheNeed((), 24))], 4, 6, 2, torch.float32, "cpu")
    with pytest.raises(EngineError):         # a budget counts each pool in its own type
        CacheManager(needs, 4, 6, 2, torch.float32, "cpu", max_bytes=6 * 4 * (24 * 2 + 15 * 4 + 32 * 4) - 1)


def test_groups_by_need_and_shared_caches():
    needs = [RunNeed(0, CacheNeed((2, 2), 8, None)), RunNeed(1, CacheNeed((2, 1), 16, 6)), RunNeed(0, CacheNeed((2, 2), 8, None)),
             RunNeed(3, None), RunNeed(4, CacheNeed((2, 2), 8, 6))]
    cache = CacheManager(needs, 4, 6, 2, torch.float32, "cpu")
    assert [group.window for group in cache.groups] == [None, 6]
    assert [b.group for b in cache.bindings] == [0, 1, 0, None, 1]
    assert cache.bindings[2].cache is cache.bindings[0].cache and not cache.bindings[2].writes and cache.bindings[0].writes
    assert cache.bindings[1].cache.shape == (6, 2, 1, 4 * 16) and cache.bindings[4].cache.shape == (6, 2, 2, 4 * 8)
    with pytest.raises(EngineError):
        CacheManager([RunNeed(0, CacheNeed((2, 2), 8)), RunNeed(0, CacheNeed((2, 1), 8))], 4, 6, 2, torch.float32, "cpu")
    # the windowed group gives pages back as the request grows; the full group keeps them
    cache.admit("a")
    for _ in range(5):
        cache.reserve("a", 4)
        cache.commit("a", 4)
        cache.check()
    assert cache.length("a") == 20
    assert cache.page_list("a", 0) == [0, 1, 2, 3, 4]
    # window 6 at length 20: a later token (position >= 20) sees keys >= 15, so blocks 0..2 (positions 0..11) are gone
    assert [page == ABSENT for page in cache.page_list("a", 1)] == [True, True, True, False, False]
    assert cache.free_pages() == [1, 4]
    with pytest.raises(EngineError):
        cache.rows("a", 1, 11, 1)
    assert len(cache.rows("a", 1, 12, 8)) == 8
    cache.release("a")
    cache.check()
    assert cache.free_pages() == [6, 6]


def test_window_edge_exactly():
    cache = manager(num_pages=8, page_size=4, window=4, runs=1)
    cache.admit("a")
    cache.reserve("a", 7)
    cache.commit("a", 7)       # next position 7 sees keys 4..7: block 0 (0..3) is dead
    assert [p == ABSENT for p in cache.page_list("a", 0)] == [True, False]
    cache.reserve("a", 1)
    cache.commit("a", 1)       # length 8: position 8 sees 5..8, block 1 still holds 5, 6, 7
    assert [p == ABSENT for p in cache.page_list("a", 0)] == [True, False]
    cache.reserve("a", 3)
    cache.commit("a", 3)       # length 11: position 11 sees 8..11, block 1 (4..7) is dead
    assert [p == ABSENT for p in cache.page_list("a", 0)] == [True, True, False]


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    window = [None, 5, None, 9, 3, None][seed]
    cache = manager(num_pages=12, page_size=4, max_requests=4, window=window, runs=2)
    live, counter = [], 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and cache.free_slots > 0:
            counter += 1
            cache.admit(counter)
            live.append(counter)
        elif action < 0.8 and live:
            request = rng.choice(live)
            count = rng.randint(1, 9)
            if cache.length(request) + count > 64:
                continue
            if cache.can_reserve([(request, count)]):
                cache.reserve(request, count)
                rows = cache.rows(request, 0, cache.length(request), count)
                assert len(set(rows)) == count
                cache.commit(request, count)
            else:
                with pytest.raises(EngineError):
                    cache.reserve(request, count)
        elif live:
            request = live.pop(rng.randrange(len(live)))
            cache.release(request)
            with pytest.raises(EngineError):
                cache.release(request)
        cache.check()
        # no row of the cache belongs to two live requests
        held = [page for request in live for page in cache.page_list(request, 0) if page != ABSENT]
        assert len(held) == len(set(held))
    for request in live:
        cache.release(request)
    cache.check()
    assert cache.free_pages() == [12] and cache.free_slots == 4


def test_a_byte_budget_refuses_a_pool_before_it_is_allocated():
    """src/kv_cache.cpp:40-43: more than the configured bytes is out_of_memory."""
    needs = [RunNeed(0, CacheNeed((2, 2), 8)), RunNeed(1, CacheNeed((2, 2), 8)), RunNeed(0, CacheNeed((2, 2), 8))]   # two pools, one reader
    per_page = CacheManager.page_bytes(needs, 4, torch.float32)
    assert per_page == 2 * (2 * 2 * 4 * 8 * 4)
    CacheManager(needs, 4, 10, 2, torch.float32, "cpu", max_bytes=10 * per_page)
    with pytest.raises(EngineError) as caught:
        CacheManager(needs, 4, 11, 2, torch.float32, "cpu", max_bytes=10 * per_page)
    assert caught.value.code == ErrorCode.OUT_OF_MEMORY and "budget" in caught.value.message
    assert CacheManager.page_bytes(needs, 4, torch.bfloat16) == per_page // 2
