"""The cache manager's bookkeeping on the CPU: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; slots carry state."""

import random

import pytest
import torch

from pagedserve_amd.cache import (CacheFull, CacheGroupSpec, CacheManager, PagePool, StateSpec,
                                  kv_cache_budget)


def _manager(pages=8, page_size=4, slots=4, window=0, states=(), groups=None, **kwargs):
    groups = groups or [CacheGroupSpec((0, 1), 2, 16, window)]
    return CacheManager(groups, pages, page_size, slots, torch.float32, "cpu", states, **kwargs)


def test_pages_follow_the_length():
    manager = _manager(page_size=2)
    manager.admit("r")
    manager.grow("r", 5)
    manager.commit("r", 5)
    # 5 tokens, pages of 2 -> 3 pages (testing/test_project.py:58-62)
    assert len(manager.table("r", 0)) == 3 and manager.length("r") == 5
    manager.grow("r", 6)
    assert len(manager.table("r", 0)) == 3       # position 5 fits the third page
    manager.commit("r", 6)
    manager.grow("r", 7)
    assert len(manager.table("r", 0)) == 4       # a token on a page boundary takes a page
    manager.commit("r", 7)
    manager.check_invariants()
    manager.release("r")
    assert manager.pools[0].num_free == 8 and not manager.requests
    manager.check_invariants()


def test_room_in_the_last_page_is_noted_and_not_exceeded():
    """The positions that a request's pages have room for are kept beside its length: growing
    inside them takes nothing, committing beyond them is an error, and a pool that runs out
    leaves them as they were."""
    manager = _manager(pages=3, page_size=4)
    manager.admit("r")
    assert manager.requests["r"].capacity == 0
    manager.grow("r", 5)
    assert manager.requests["r"].capacity == 8 and manager.pools[0].num_free == 1
    manager.grow("r", 8)
    assert manager.pools[0].num_free == 1
    with pytest.raises(RuntimeError, match="beyond the pages"):
        manager.commit("r", 9)
    manager.commit("r", 8)
    manager.admit("s")
    manager.grow("s", 4)
    with pytest.raises(CacheFull):
        manager.grow("r", 9)
    assert manager.requests["r"].capacity == 8
    manager.check_invariants()
    manager.requests["r"].capacity = 12         # a wrong note is found
    with pytest.raises(AssertionError, match="room for 12"):
        manager.check_invariants()


def test_prompt_of_four_with_pages_of_four():
    # prompt 4, page 4 -> 2 pages after one decoded token (testing/test_project.py:709-710)
    manager = _manager(page_size=4)
    manager.admit("r")
    manager.grow("r", 4)
    manager.commit("r", 4)
    assert len(manager.table("r", 0)) == 1
    manager.grow("r", 5)
    manager.commit("r", 5)
    assert len(manager.table("r", 0)) == 2


def test_lifo_reuse_and_disjoint_tables():
    manager = _manager(pages=6, page_size=4)
    manager.admit("a")
    manager.grow("a", 8)
    manager.commit("a", 8)
    first = list(manager.table("a", 0))
    manager.admit("b")
    manager.grow("b", 4)
    assert not set(first) & set(manager.table("b", 0))
    manager.commit("b", 4)
    manager.release("a")
    manager.admit("c")
    manager.grow("c", 4)
    # a page that was just freed is handed out next (src/model/kv_manager.py:118,127)
    assert manager.table("c", 0)[0] in first
    manager.check_invariants()


def test_full_cache_rolls_back():
    manager = _manager(pages=3, page_size=4)
    manager.admit("a")
    manager.grow("a", 8)
    manager.commit("a", 8)
    manager.admit("b")
    with pytest.raises(CacheFull, match="KV cache full"):
        manager.grow("b", 9)                     # needs 3, one is free
    assert manager.pools[0].num_free == 1 and manager.table("b", 0) == []
    assert not manager.can_grow("b", 9) and manager.can_grow("b", 4)
    manager.check_invariants()


def test_double_free_and_unknown_requests_raise():
    pool = PagePool(2)
    page = pool.allocate()
    pool.free(page)
    with pytest.raises(RuntimeError, match="freed twice"):
        pool.free(page)
    manager = _manager()
    with pytest.raises(RuntimeError, match="not live"):
        manager.release("ghost")
    manager.admit("a")
    with pytest.raises(RuntimeError, match="already live"):
        manager.admit("a")
    with pytest.raises(ValueError, match="shrink"):
        manager.grow("a", 4)
        manager.commit("a", 4)
        manager.grow("a", 2)
    with pytest.raises(RuntimeError, match="beyond the pages"):
        manager.commit("a", 100)


def test_slots_run_out_and_come_back():
    manager = _manager(slots=2)
    first, second = manager.admit("a"), manager.admit("b")
    assert first != second
    with pytest.raises(CacheFull, match="slot"):
        manager.admit("c")
    manager.release("a")
    assert manager.admit("c") == first


def test_state_slots_are_zeroed_on_admission():
    manager = _manager(states=[StateSpec(entry=1, shape=(3, 2))], groups=[CacheGroupSpec((0,), 1, 16)])
    slot = manager.admit("a")
    assert manager.state(1).shape == (4, 3, 2)
    manager.state(1)[slot] += 5.0
    manager.release("a")
    again = manager.admit("b")
    assert again == slot and float(manager.state(1)[again].abs().max()) == 0.0


def test_window_group_gives_pages_back_early():
    groups = [CacheGroupSpec((0,), 1, 16, 0), CacheGroupSpec((1,), 1, 16, window=6)]
    manager = CacheManager(groups, [16, 16], 4, 2, torch.float32, "cpu")
    manager.admit("r")
    length = 0
    for step in (5, 1, 1, 7, 1, 1, 1, 9):
        manager.grow("r", length + step)
        length += step
        manager.commit("r", length)
        full, windowed = manager.table("r", 0), manager.table("r", 1)
        assert len(full) == -(-length // 4) and all(page >= 0 for page in full)
        # the next query (position `length`) sees keys > length - 6: their pages must be held,
        # and every page wholly at or before length - 6 must be back in the pool
        for index, page in enumerate(windowed):
            last_position = index * 4 + 3
            if last_position <= length - 6:
                assert page == -1, (length, index)
            else:
                assert page >= 0, (length, index)
        manager.check_invariants()
    assert manager.pools[1].num_allocated <= 3 and manager.pools[0].num_allocated == 7
    assert manager.pages_for_length(1, 1000, longest_step=9) == -(-(6 + 9) // 4) + 1
    assert manager.pages_for_length(0, 1000) == 250
    manager.release("r")
    assert manager.pools[0].num_free == 16 and manager.pools[1].num_free == 16


def test_groups_have_pools_of_their_own():
    groups = [CacheGroupSpec((0, 2), 2, 16), CacheGroupSpec((1,), 4, 32)]
    manager = CacheManager(groups, [5, 7], 8, 2, torch.bfloat16, "cpu")
    assert manager.key_pools[0].shape == (2, 5, 2, 8, 16) and manager.value_pools[1].shape == (1, 7, 4, 8, 32)
    k, v = manager.entry_pools(2)
    assert k.data_ptr() == manager.key_pools[0][1].data_ptr() and k.shape == (5, 2, 8, 16)
    assert manager.entry_group(1) == 1
    # bytes per page: 2 (K and V) x entries x heads x page x head_dim x element size
    # (src/model/kv_manager.py:55-58)
    assert manager.bytes_per_page(0) == 2 * 2 * 2 * 8 * 16 * 2
    with pytest.raises(ValueError, match="two groups"):
        CacheManager([CacheGroupSpec((0,), 1, 16), CacheGroupSpec((0,), 1, 16)], 4, 4, 1, torch.float32, "cpu")


def test_usage_summary_tracks_peak():
    # testing/test_memory_budget.py:50-73: 4 pages, peak 2, all free at the end
    manager = CacheManager([CacheGroupSpec((0,), 1, 2)], 4, 2, 2, torch.float32, "cpu")
    manager.reset_usage_stats()
    manager.admit("a")
    manager.grow("a", 4)
    manager.commit("a", 4)
    manager.release("a")
    summary = manager.usage_summary()["groups"][0]
    per_page = 2 * 1 * 1 * 2 * 2 * 4
    assert summary == {"total_blocks": 4, "free_blocks_at_end": 4, "peak_allocated_blocks": 2,
                       "peak_allocated_tokens": 4, "peak_allocated_bytes": per_page * 2,
                       "peak_utilization_percent": 50, "bytes_per_block": per_page,
                       "bytes_per_token": per_page // 2}


def test_budget_rule():
    # testing/test_memory_budget.py:8-23
    assert kv_cache_budget(800, 1000, 0.8, 100) == 600
    assert kv_cache_budget(800, 1000, 0.9, 150) == 650
    for kwargs in ({"memory_utilization": 0}, {"memory_utilization": 1.1}, {"safety_memory": -1}):
        with pytest.raises(ValueError):
            kv_cache_budget(800, 1000, **kwargs)
    with pytest.raises(ValueError):
        kv_cache_budget(0, 1000)
    with pytest.raises(ValueError):
        kv_cache_budget(1100, 1000)
    with pytest.raises(RuntimeError):
        kv_cache_budget(100, 1000, safety_memory=200)


@pytest.mark.parametrize("seed", range(8))
@pytest.mark.parametrize("window", [0, 10])
def test_random_orders_keep_the_invariants(seed, window):
    rng = random.Random(seed)
    groups = [CacheGroupSpec((0,), 1, 16, 0), CacheGroupSpec((1,), 1, 16, window)]
    manager = CacheManager(groups, [24, 24], 4, 5, torch.float32, "cpu", max_positions=64)
    lengths = {}
    next_id = 0
    for _ in range(400):
        action = rng.random()
        if action < 0.25 and len(lengths) < 5:
            manager.admit(next_id)
            lengths[next_id] = 0
            next_id += 1
        elif action < 0.85 and lengths:
            rid = rng.choice(list(lengths))
            step = rng.choice([1, 1, 1, 2, 5, 13])
            if lengths[rid] + step > 64:
                continue
            try:
                manager.grow(rid, lengths[rid] + step)
            except CacheFull:
                manager.check_invariants()
                victim = rng.choice(list(lengths))
                manager.release(victim)
                del lengths[victim]
                continue
            if rng.random() < 0.1:
                continue                          # a step that failed: pages stay, length does not move
            lengths[rid] += step
            manager.commit(rid, lengths[rid])
        elif lengths:
            rid = rng.choice(list(lengths))
            manager.release(rid)
            del lengths[rid]
        manager.check_invariants()
        for rid, length in lengths.items():
            assert manager.length(rid) == length
            assert len(manager.table(rid, 0)) >= -(-length // 4)
    for rid in list(lengths):
        manager.release(rid)
    manager.check_invariants()
    assert all(pool.num_free == pool.num_pages for pool in manager.pools)
    assert len(manager.free_slots) == 5


def test_values_may_have_another_head_size_than_keys():
    """A group whose values are narrower than its keys: the value pool has its own last
    dimension, a page's bytes count both, and groups that differ only in that are different
    groups."""
    wide = CacheGroupSpec((0,), 2, 16, 0, value_dim=8)
    same = CacheGroupSpec((1,), 2, 16)
    assert wide.value_head_dim == 8 and same.value_head_dim == 16
    assert wide.geometry() != same.geometry()
    manager = CacheManager([wide, same], 5, 4, 2, torch.float32, "cpu")
    keys, values = manager.entry_pools(0)
    assert keys.shape == (5, 2, 4, 16) and values.shape == (5, 2, 4, 8)
    keys, values = manager.entry_pools(1)
    assert keys.shape == values.shape == (5, 2, 4, 16)
    assert manager.bytes_per_page(0) == 2 * 4 * (16 + 8) * 4
    assert manager.bytes_per_page(1) == 2 * 4 * (16 + 16) * 4
