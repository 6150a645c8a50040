"""The cache manager (CPU): no page lost, held twice or freed twice, under random
orders of requests; windows give pages back; prefixes are shared by reference count."""
import random

import pytest

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import (CacheError, CacheManager, GroupSpec, OutOfPages, PagePool, StateSlots,
                                   chain_hash, plan_cache, KVNeed, StateNeed)


def test_pages_are_handed_out_from_zero_and_reused_last_in_first_out():
    pool = PagePool(4)                                   # reference kvcache.py:67,152,166
    assert [pool.allocate() for _ in range(3)] == [0, 1, 2]
    pool.release(1)
    pool.release(0)
    assert pool.allocate() == 0 and pool.allocate() == 1 and pool.allocate() == 3
    with pytest.raises(OutOfPages):
        pool.allocate()


def test_a_scattered_pool_hands_out_every_page_once_in_a_fixed_order():
    """The scattered order is a permutation of the pages, the same in every pool of that size, and not the
    order 0, 1, 2, ...; pages that come back are reused last in, first out as in the plain pool."""
    a, b = PagePool(257, scatter=True), PagePool(257, scatter=True)
    order = [a.allocate() for _ in range(257)]
    assert sorted(order) == list(range(257)) and order != list(range(257))
    assert [b.allocate() for _ in range(257)] == order
    with pytest.raises(OutOfPages):
        a.allocate()
    a.release(order[5])
    a.release(order[9])
    assert a.allocate() == order[9] and a.allocate() == order[5]
    # aligned runs of neighbouring pages stay together and in order; the runs lie at no regular distances
    run = PagePool.SCATTER_RUN
    c = PagePool(32 * run, scatter=True)
    order = [c.allocate() for _ in range(32 * run)]
    starts = order[::run]
    assert sorted(order) == list(range(32 * run)) and all(s % run == 0 for s in starts)
    assert all(order[i:i + run] == list(range(order[i], order[i] + run)) for i in range(0, 32 * run, run))
    assert len({b - a for a, b in zip(starts, starts[1:])}) > 16
    m = CacheManager([GroupSpec(), GroupSpec(window=8)], [64, 64], page_size=4, max_requests=2, scatter_pages=True)
    m.add_request("r")
    m.reserve("r", 40)
    m.commit("r", list(range(40)))
    m.check_invariants()
    m.free_request("r")
    assert all(pool.num_free == 64 for pool in m.pools)


def test_reference_counts_refuse_misuse():
    pool = PagePool(2)
    p = pool.allocate()
    pool.retain(p)
    assert not pool.release(p) and pool.release(p)
    with pytest.raises(CacheError):
        pool.release(p)                                  # freed twice
    with pytest.raises(CacheError):
        pool.retain(p)                                   # retain of a free page
    with pytest.raises(CacheError):
        pool.retain(7)


def test_state_slots():
    s = StateSlots(2)
    a, b = s.take("a"), s.take("b")
    assert {a, b} == {0, 1}
    with pytest.raises(CacheError):
        s.take("c")
    s.give_back(a)
    with pytest.raises(CacheError):
        s.give_back(a)
    assert s.take("c") == a


def test_reserve_is_all_or_nothing_and_commit_needs_pages():
    m = CacheManager([GroupSpec()], 4, page_size=4, max_requests=2)
    m.add_request("a")
    m.reserve("a", 9)                                    # 3 pages
    assert m.block_table("a", 0) == [0, 1, 2]
    m.add_request("b")
    with pytest.raises(OutOfPages):
        m.reserve("b", 5)                                # needs 2, 1 free
    assert m.block_table("b", 0) == [] and m.num_free_pages() == 1
    assert not m.can_reserve([("b", 5)]) and m.can_reserve([("b", 4)])
    with pytest.raises(CacheError):
        m.commit("b", [1, 2, 3])                         # nothing reserved
    m.commit("a", list(range(9)))
    assert m.token_slots("a", 0, 7, 2) == [1 * 4 + 3, 2 * 4 + 0]
    m.free_request("a")
    assert m.num_free_pages() == 4
    with pytest.raises(CacheError):
        m.free_request("a")
    m.check_invariants()


def test_window_group_gives_pages_back_once_passed():
    P, W = 4, 6
    m = CacheManager([GroupSpec(), GroupSpec(window=W)], [16, 16], page_size=P, max_requests=1)
    m.add_request(0)
    n = 0
    for step in (5, 3, 1, 1, 1, 8, 1, 1):
        m.reserve(0, n + step)
        # every key a query of this step can see has a page
        for pos in range(n, n + step):
            for key in range(max(0, pos - W + 1), pos + 1):
                assert m.block_table(0, 1)[key // P] >= 0
        m.commit(0, [1] * step)
        n += step
        full, win = m.block_table(0, 0), m.block_table(0, 1)
        assert all(p >= 0 for p in full)
        first_live = max(0, n - W + 1) // P              # the next query is at position n
        assert all(p < 0 for p in win[:first_live]) and all(p >= 0 for p in win[first_live:])
        m.check_invariants()
    held = sum(p >= 0 for p in m.block_table(0, 1))
    assert held <= (W + P - 1) // P + 1
    assert m.pools[1].num_free == 16 - held


def test_random_orders_keep_every_invariant():
    rng = random.Random(0)
    for trial in range(30):
        P = rng.choice([1, 4, 8])
        groups = [GroupSpec()] if trial % 2 else [GroupSpec(), GroupSpec(window=rng.choice([3, 9, 17]))]
        m = CacheManager(groups, rng.choice([6, 12, 40]), page_size=P, max_requests=4,
                         prefix_sharing=(trial % 2 == 1), keep_freed_prefixes=(trial % 4 == 3))
        live, next_id = {}, 0
        common = [rng.randrange(50) for _ in range(3 * P)]
        for _ in range(200):
            op = rng.random()
            if op < 0.25 and len(live) < 4:
                prompt = (common if rng.random() < 0.6 else []) + [rng.randrange(50) for _ in range(rng.randrange(1, 20))]
                m.add_request(next_id)
                start = m.match_prefix(next_id, prompt)
                assert start % P == 0 and start < len(prompt)
                live[next_id] = (prompt, start)
                next_id += 1
            elif op < 0.85 and live:
                rid = rng.choice(list(live))
                prompt, done = live[rid]
                if done < len(prompt):
                    n = rng.randrange(1, len(prompt) - done + 1)
                    toks = prompt[done:done + n]
                else:
                    n, toks = 1, [rng.randrange(50)]
                    prompt = prompt + toks
                if m.can_reserve([(rid, done + n)]):
                    m.reserve(rid, done + n)
                    m.commit(rid, toks)
                    live[rid] = (prompt, done + n)
                else:
                    with pytest.raises(OutOfPages):
                        m.reserve(rid, done + n)
            elif live:
                rid = rng.choice(list(live))
                m.free_request(rid)
                del live[rid]
            m.check_invariants()
        for rid in list(live):
            m.free_request(rid)
        m.check_invariants()
        assert all(m.available(g) == pool.num_pages for g, pool in enumerate(m.pools))   # free, or kept and free to take
        if m.keep_freed:
            assert len(m._shared) == len(m._kept) == len(m._page_hash)
            m.reset()
            m.check_invariants()
        assert all(pool.num_free == pool.num_pages for pool in m.pools)
        assert not m._shared and not m._page_hash and not m._kept


def test_prefix_is_shared_by_full_pages_only_and_one_token_is_left():
    P = 4
    m = CacheManager([GroupSpec()], 16, page_size=P, max_requests=3, prefix_sharing=True)
    prompt = list(range(10, 22))                         # 12 tokens = 3 full pages
    m.add_request("a")
    assert m.match_prefix("a", prompt) == 0
    m.reserve("a", 6)
    m.commit("a", prompt[:6])                            # page 0 full and registered, page 1 half
    m.add_request("b")
    assert m.match_prefix("b", prompt) == 4              # only what is computed can be shared
    assert m.block_table("b", 0) == [m.block_table("a", 0)[0]]
    m.reserve("a", 12)
    m.commit("a", prompt[6:])
    m.add_request("c")
    assert m.match_prefix("c", prompt) == 8              # 12 tokens match, but one must be computed
    assert m.get("c").shared_len == 8
    assert m.pools[0].refcount[m.block_table("a", 0)[0]] == 3
    m.check_invariants()
    m.free_request("a")                                  # pages survive while b and c hold them
    m.check_invariants()
    assert m.pools[0].refcount[m.block_table("c", 0)[1]] == 1
    m.free_request("b")
    m.free_request("c")
    m.check_invariants()
    assert m.num_free_pages() == 16 and not m._shared   # a freed page leaves the registry
    m.add_request("d")
    assert m.match_prefix("d", prompt) == 0


def test_freed_prefixes_are_kept_until_their_memory_is_needed():
    P = 2
    m = CacheManager([GroupSpec()], 8, page_size=P, max_requests=2, prefix_sharing=True, keep_freed_prefixes=True)
    prompt = [1, 2, 3, 4, 5, 6, 7]                       # 3 full pages and one token
    m.add_request("a")
    m.reserve("a", 7)
    m.commit("a", prompt)
    pages_a = list(m.block_table("a", 0))
    m.free_request("a")
    m.check_invariants()
    assert m.pools[0].num_free == 5 and m.available() == 8          # three pages kept, one freed
    assert all(m.pools[0].refcount[p] == 0 for p in pages_a)
    # a later request with the same beginning takes the kept pages over
    m.add_request("b")
    assert m.match_prefix("b", prompt) == 6
    assert m.block_table("b", 0) == pages_a[:3] and m.stats["kept_page_hits"] == 3
    assert all(m.pools[0].refcount[p] == 1 for p in pages_a[:3])
    m.check_invariants()
    m.free_request("b")
    assert len(m._kept) == 3
    # a reservation that needs more than the free pages takes kept ones: the last page of the prefix first
    m.add_request("c")
    m.reserve("c", 12)                                   # 6 pages: 5 free + 1 kept
    m.check_invariants()
    assert m.stats["kept_pages_evicted"] == 1 and len(m._kept) == 2
    assert pages_a[2] in m.block_table("c", 0) and pages_a[0] not in m.block_table("c", 0)
    m.add_request("d")
    assert m.match_prefix("d", prompt) == 4              # the first two pages are still there
    assert not m.can_reserve([("d", 7)])                 # nothing free, nothing kept
    with pytest.raises(OutOfPages):
        m.reserve("d", 7)
    m.free_request("c")
    m.free_request("d")
    m.check_invariants()
    m.reset()
    assert m.pools[0].num_free == 8 and not m._shared and not m._kept


def test_a_different_token_breaks_the_chain():
    assert chain_hash(0, [1, 2, 3]) != chain_hash(0, [1, 2, 4])
    assert chain_hash(5, [1, 2, 3]) != chain_hash(0, [1, 2, 3])
    assert chain_hash(0, [1, 2, 3]) == chain_hash(0, (1, 2, 3))
    m = CacheManager([GroupSpec()], 8, page_size=2, max_requests=2, prefix_sharing=True)
    m.add_request("a")
    m.reserve("a", 6)
    m.commit("a", [1, 2, 3, 4, 5, 6])
    m.add_request("b")
    assert m.match_prefix("b", [1, 2, 9, 4, 5, 6, 7]) == 2   # page 1 differs: page 2 cannot match either


def test_sharing_is_off_when_a_group_has_a_window():
    m = CacheManager([GroupSpec(), GroupSpec(window=4)], 8, page_size=2, max_requests=2, prefix_sharing=True)
    assert not m.prefix_sharing


def test_plan_groups_entries_by_need_and_lets_an_entry_read_another():
    full = KVNeed(2, 16, None)
    win = KVNeed(2, 16, 8)
    plan = plan_cache([(full, None, None), (win, None, None), (full, None, 0), (None, StateNeed((4,)), None),
                       (win, None, None)])
    assert plan.groups == [GroupSpec(None), GroupSpec(8)]
    assert plan.user_group == [0, 1, 0, None, 1]
    assert plan.user_source == [0, 1, 0, None, 4]
    assert plan.user_kv[2] is None and plan.user_state[3] == StateNeed((4,))
    assert plan.bytes_per_token(2) == 3 * 2 * 2 * 16 * 2
    with pytest.raises(ValueError):
        plan_cache([(full, None, None), (KVNeed(1, 16, None), None, 0)])


def test_an_entry_cannot_read_a_cache_that_keeps_fewer_keys_than_it_sees():
    """The source's group gives pages back once its window has passed them: a reader over all keys,
    or with a wider window, would follow table entries that are -1 by then."""
    kv = lambda w: KVNeed(num_kv_heads=2, head_dim=16, window=w)
    plan_cache([(kv(None), None, None), (kv(8), None, 0)])          # a window over a cache of all keys
    plan_cache([(kv(16), None, None), (kv(16), None, 0), (kv(5), None, 0)])
    with pytest.raises(ValueError):
        plan_cache([(kv(16), None, None), (kv(None), None, 0)])
    with pytest.raises(ValueError):
        plan_cache([(kv(16), None, None), (kv(17), None, 0)])


def test_pages_handed_out_and_given_back_are_noted_and_kept_pages_are_not():
    """What the owner of the storage overwrites in its debug mode: every page that leaves or
    reaches a free list, never a page that is kept for a later request with the same prefix."""
    m = CacheManager([GroupSpec(), GroupSpec(window=6)], 6, page_size=4, max_requests=2,
                     prefix_sharing=False)
    m.track_pages = True
    m.add_request("a")
    m.reserve("a", 10)
    assert sorted(m.take_page_events()) == [(0, 0), (0, 1), (0, 2), (1, 0), (1, 1), (1, 2)]
    m.commit("a", list(range(10)))                       # the window of 6 has passed positions 0..3
    assert m.take_page_events() == [(1, 0)]
    m.free_request("a")
    assert sorted(m.take_page_events()) == [(0, 0), (0, 1), (0, 2), (1, 1), (1, 2)]
    assert m.take_page_events() == []
    # kept prefixes: a finished request's registered pages stay, and are noted only when evicted
    k = CacheManager([GroupSpec()], 3, page_size=4, max_requests=2, prefix_sharing=True, keep_freed_prefixes=True)
    k.track_pages = True
    k.add_request("a")
    k.reserve("a", 9)
    k.commit("a", list(range(9)))
    k.take_page_events()
    k.free_request("a")                                  # pages 0 and 1 are full and registered: kept
    assert k.take_page_events() == [(0, 2)] and k.num_kept == 2
    k.add_request("b")
    k.reserve("b", 12)                                   # needs all three pages: the kept ones are given up
    ev = k.take_page_events()
    assert sorted(set(ev)) == [(0, 0), (0, 1), (0, 2)] and k.num_kept == 0
    k.check_invariants()


def test_plan_with_blocks_of_several_cache_users_and_of_none():
    """A block says how many of its parts keep something per request: two mixers side by side are two
    users of one schedule entry, a block without a mixer has none; an entry that reads another entry's
    cache pairs its users with that entry's."""
    full, win = KVNeed(2, 16, None), KVNeed(2, 16, 8)
    plan = plan_cache([([(full, None), (win, StateNeed((3,)))], None),     # entry 0: users 0 and 1
                       ([], None),                                           # entry 1: no user
                       ([(full, None), (win, None)], 0),                     # entry 2: reads entry 0's two caches
                       (full, None, None)])                                  # entry 3: the short form, one user
    assert plan.entry_users == [[0, 1], [], [2, 3], [4]]
    assert plan.groups == [GroupSpec(None), GroupSpec(8)]
    assert plan.user_group == [0, 1, 0, 1, 0]
    assert plan.user_source == [0, 1, 0, 1, 4]
    assert plan.user_kv == [full, win, None, None, full]
    assert plan.user_state == [None, StateNeed((3,)), None, None, None]
    with pytest.raises(ValueError):
        plan_cache([([(full, None), (win, None)], None), ([(full, None)], 0)])   # one user cannot pair with two
