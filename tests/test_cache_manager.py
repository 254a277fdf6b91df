"""The cache manager on the host: no page lost, held twice or freed twice,
under random orders of requests; windows give pages back; slots."""
import random

import pytest

from inferx_amd.cache.manager import (RESERVE_CONTEXT_FULL, RESERVE_OK, RESERVE_POOL_EMPTY, CacheError, CacheManager,
                                      GroupLayout, PagePool, pages_for_window)
from inferx_amd.engine.batch import BatchError, build_step_batch


def test_pool_lifo_and_double_free():
    pool = PagePool(3)
    assert [pool.allocate() for _ in range(3)] == [0, 1, 2]  # page 0 first (reference: kv_cache.cc:58-64)
    assert pool.allocate() is None
    pool.release(1)
    with pytest.raises(CacheError):
        pool.release(1)
    with pytest.raises(CacheError):
        pool.release(7)
    assert pool.allocate() == 1 and pool.free_pages == 0


def test_reserve_commit_free():
    m = CacheManager([GroupLayout(0)], [4], page_size=4, max_requests=2, max_seq_len=16)
    m.add("a")
    assert m.reserve("a", 5) == RESERVE_OK and m.pools[0].used_pages == 2  # 5 tokens: two pages of 4
    assert m.slot_index("a", 0, 4) == m.block_row("a", 0)[1] * 4
    m.commit("a", 5)
    assert m.cached("a") == 5
    with pytest.raises(CacheError):
        m.commit("a", 1)  # nothing reserved beyond 5
    assert m.reserve("a", 17) == RESERVE_CONTEXT_FULL
    m.add("b")
    assert m.reserve("b", 9) == RESERVE_POOL_EMPTY and m.pools[0].used_pages == 2  # all or nothing
    assert m.reserve("b", 8) == RESERVE_OK and m.pools[0].free_pages == 0
    with pytest.raises(CacheError):
        m.add("c")  # no slot left
    m.free("a")
    assert m.pools[0].free_pages == 2
    with pytest.raises(CacheError):
        m.free("a")
    m.free("b")
    m.check()
    assert m.pools[0].used_pages == 0


def test_groups_have_pages_of_their_own():
    m = CacheManager([GroupLayout(0), GroupLayout(8)], [8, 3], page_size=4, max_requests=2, max_seq_len=32)
    m.add("a")
    assert m.reserve("a", 12) == RESERVE_OK
    assert m.pools[0].used_pages == 3 and m.pools[1].used_pages == 3
    m.commit("a", 12)
    # next query is at position 12, window 8 reads keys 5..12: page 0 (tokens 0..3) is dead
    assert m.block_row("a", 1)[0] == -1 and m.pools[1].used_pages == 2
    assert m.block_row("a", 0)[0] >= 0  # the full group keeps everything
    # the windowed pool has 3 pages, yet the request grows on: a passed page comes back for each new one
    for n in range(13, 33):
        assert m.reserve("a", n) == RESERVE_OK, n
        m.commit("a", 1)
        m.check()
        assert m.pools[1].used_pages <= 3
    assert m.pools[0].used_pages == 8
    with pytest.raises(CacheError):
        m.slot_index("a", 1, 3)  # given back
    m.free("a")
    m.check()
    assert all(p.used_pages == 0 for p in m.pools)


def test_window_rule_exactly():
    # page j is dead once (j + 1) * P <= cached + 1 - W
    m = CacheManager([GroupLayout(5)], [16], page_size=4, max_requests=1, max_seq_len=64)
    m.add("a")
    m.reserve("a", 8)
    m.commit("a", 8)   # next p = 8 reads 4..8 -> page 0 dead
    assert m.block_row("a", 0)[:2] == [-1, m.block_row("a", 0)[1]] and m.block_row("a", 0)[1] >= 0
    m.reserve("a", 12)
    m.commit("a", 3)   # cached 11, next p = 11 reads 7..11 -> page 1 (4..7) still read
    assert m.block_row("a", 0)[1] >= 0
    m.commit("a", 1)   # cached 12, reads 8..12 -> page 1 dead
    assert m.block_row("a", 0)[1] == -1


def test_a_windowed_group_may_keep_every_page():
    # the switch for differential tests: the same window, but passed pages stay until the request ends
    keep = CacheManager([GroupLayout(5, release_passed=False)], [16], page_size=4, max_requests=1, max_seq_len=64)
    give = CacheManager([GroupLayout(5)], [16], page_size=4, max_requests=1, max_seq_len=64)
    for m in (keep, give):
        m.add("a")
        m.reserve("a", 40)
        m.commit("a", 40)
    assert keep.groups[0].window == 5 and keep.pools[0].used_pages == 10 and -1 not in keep.block_row("a", 0)[:10]
    # the next query, at position 40, reads keys 36..40: pages 0..8 (tokens 0..35) are dead
    assert give.pools[0].used_pages == 1 and give.block_row("a", 0)[:9] == [-1] * 9
    for m in (keep, give):
        m.free("a")
        m.check()
        assert m.pools[0].used_pages == 0


def test_a_windowed_group_takes_pages_as_the_steps_reach_them():
    # window 8, pages of 4, steps of at most 6 tokens: whatever is reserved, the windowed group holds the pages
    # for the window behind and one step ahead, the full group everything
    per_request = pages_for_window(8, 4, 1, 6)
    assert per_request == 6  # ceil((8 + 6) / 4) + 2
    m = CacheManager([GroupLayout(0), GroupLayout(8)], [32, per_request], page_size=4, max_requests=1, max_seq_len=128,
                     max_step_tokens=6)
    m.add("a")
    assert m.reserve("a", 100) == RESERVE_OK          # a long prompt, reserved whole (as a scheduler admits it)
    assert m.pools[0].used_pages == 25 and m.pools[1].used_pages == 2   # 6 tokens ahead: 2 pages
    fed = 0
    while fed < 100:
        n = min(6, 100 - fed)
        batch = build_step_batch(m, [("a", [1] * n, [])])
        assert batch.slots[1].min() >= 0 and m.pools[1].used_pages <= per_request
        batch.validate(10, [p.num_pages for p in m.pools], 4)           # every slot under its table, both groups
        m.commit("a", n)
        fed += n
        m.check()
    assert m.pools[0].used_pages == 25 and m.pools[1].used_pages <= 3
    with pytest.raises(BatchError, match="6 at most"):
        m.reserve("a", 120)
        build_step_batch(m, [("a", [1] * 7, [])])
    m.free("a")
    assert all(p.used_pages == 0 for p in m.pools)
    # without the promise of a largest step the windowed group holds what is reserved, as before
    m = CacheManager([GroupLayout(8)], [32], page_size=4, max_requests=1, max_seq_len=128)
    m.add("a")
    m.reserve("a", 100)
    assert m.pools[0].used_pages == 25


@pytest.mark.parametrize("seed", range(4))
def test_a_windowed_pool_of_the_computed_size_never_runs_out(seed):
    rng = random.Random(seed)
    window, page, slots, cap = 24, 8, 5, 20
    m = CacheManager([GroupLayout(0), GroupLayout(window)], [400, pages_for_window(window, page, slots, cap)],
                     page_size=page, max_requests=slots, max_seq_len=600, max_step_tokens=cap)
    live = {}
    for i in range(800):
        if len(live) < slots and rng.random() < 0.3:
            rid = f"r{i}"
            m.add(rid)
            target = rng.randint(1, 600)
            if m.reserve(rid, target) == RESERVE_OK:  # (only the full group can refuse)
                live[rid] = [0, target]
            else:
                m.free(rid)
        for rid in list(live):
            done, target = live[rid]
            n = min(rng.randint(1, cap), target - done)
            build_step_batch(m, [(rid, [0] * n, [])])  # raises if any group is out of pages
            m.commit(rid, n)
            live[rid][0] = done + n
            if done + n == target:
                m.free(rid)
                del live[rid]
        m.check()
    for rid in live:
        m.free(rid)
    assert all(p.used_pages == 0 for p in m.pools)


def test_reset_keeps_the_slot():
    m = CacheManager([GroupLayout(0)], [4], 4, 2, 16)
    slot = m.add("a")
    m.reserve("a", 9)
    m.commit("a", 9)
    m.reset("a")
    assert m.cached("a") == 0 and m.pools[0].used_pages == 0 and m.slot_of("a") == slot
    m.check()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_lose_nothing(seed):
    rng = random.Random(seed)
    m = CacheManager([GroupLayout(0), GroupLayout(24)], [40, 12], page_size=8, max_requests=5, max_seq_len=200)
    live, next_id = {}, 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and m.can_add():
            m.add(next_id)
            live[next_id] = 0
            next_id += 1
        elif op < 0.80 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 7, 30])
            status = m.reserve(rid, live[rid] + n)
            if status == RESERVE_OK:
                m.commit(rid, n)
                live[rid] += n
                assert m.cached(rid) == live[rid]
            elif status == RESERVE_POOL_EMPTY and rng.random() < 0.5:
                m.reset(rid)
                live[rid] = 0
        elif op < 0.95 and live:
            rid = rng.choice(list(live))
            m.free(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free(rid)
    m.check()
    assert all(p.used_pages == 0 for p in m.pools)
