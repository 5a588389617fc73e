"""The cache manager's books: no page lost, held twice or freed twice, under random orders of
requests; windows give pages back; state slots follow the requests.  Host-only."""
import random

import pytest
import torch

from nanoinfer_amd.cache.block_manager import BlockManager, OutOfPages, PageError
from nanoinfer_amd.cache.manager import CacheError, KVCacheManager, StateSlots
from nanoinfer_amd.parts.base import CacheNeed, KVNeed, StateNeed


def full(n_caches=2, kvh=2, hd=16):
    return {c: CacheNeed(kv=KVNeed(kvh, hd)) for c in range(n_caches)}


# ------------------------------------------------------------------ page ids

def test_block_manager_order_and_reuse():
    bm = BlockManager(4)
    assert bm.allocate(2) == [0, 1]               # test/test_engine/test_block_manager.cpp:159-175
    bm.free([1])
    assert bm.allocate(1) == [1]                  # LIFO: the page freed last is handed out next
    bm.free([0])
    assert bm.allocate(3) == [0, 2, 3]
    assert bm.num_free == 0 and bm.utilization() == 1.0


def test_block_manager_all_or_nothing_and_double_free():
    bm = BlockManager(3)
    a = bm.allocate(2)
    with pytest.raises(OutOfPages):
        bm.allocate(2)
    assert bm.num_free == 1                        # the failed call changed nothing
    bm.free(a)
    with pytest.raises(PageError):
        bm.free([a[0]])                            # freed twice
    with pytest.raises(PageError):
        bm.free([7])                               # foreign id
    b = bm.allocate(1)
    with pytest.raises(PageError):
        bm.free([b[0], b[0]])                      # twice in one call: nothing is freed
    assert bm.is_taken(b[0]) and bm.num_free == 2
    bm.reset()
    assert bm.num_free == 3 and bm.allocate(1) == [0]


def test_block_manager_scattered_ids():
    """With ``scatter`` the ids come in a fixed pseudo-random order: every id once, the same order for the
    same pool (also after a reset), not the ascending one, and a freed id is still the next one out."""
    bm = BlockManager(64, scatter=True)
    first = bm.allocate(64)
    assert sorted(first) == list(range(64)) and first != list(range(64))
    assert max(b - a for a, b in zip(first, first[1:])) > 1 and bm.num_free == 0
    with pytest.raises(OutOfPages):
        bm.allocate(1)
    bm.free([first[5], first[9]])
    assert bm.allocate(1) == [first[9]] and bm.is_taken(first[9]) and not bm.is_taken(first[5])
    with pytest.raises(PageError):
        bm.free([first[5]])
    bm.reset()
    assert bm.allocate(64) == first == BlockManager(64, scatter=True).allocate(64)
    assert BlockManager(65, scatter=True).allocate(64) != first           # the order belongs to the pool's size


# ------------------------------------------------------------------ reserve / release

def test_pages_follow_tokens():
    m = KVCacheManager(full(), page_size=16, num_pages=8, max_requests=4)
    assert len(m.groups) == 1 and m.groups[0].cache_ids == [0, 1]        # same need, one group, one table
    assert m.reserve("a", 17) and m.block_table(0, "a") == [0, 1]        # ceil(17 / 16)
    assert m.reserve("a", 32) and m.block_table(0, "a") == [0, 1]        # still inside the second page
    assert m.reserve("a", 33) and m.block_table(0, "a") == [0, 1, 2]
    assert m.num_tokens("a") == 33 and m.free_pages() == 5
    assert m.reserve("b", 1) and m.block_table(0, "b") == [3]
    assert not m.reserve("b", 16 * 5 + 1)                                # five more pages, four free
    assert m.block_table(0, "b") == [3] and m.num_tokens("b") == 1       # unchanged by the refusal
    m.check()
    m.release("a")
    assert m.free_pages() == 7
    assert m.reserve("c", 40) and m.block_table(0, "c") == [2, 1, 0]     # handed out again, last freed first
    with pytest.raises(CacheError):
        m.release("a")
    with pytest.raises(CacheError):
        m.reserve("c", 10)                                               # a request does not shrink
    m.check()
    m.reset()
    assert m.free_pages() == 8 and not m.live_requests()


def test_can_reserve_all_counts_the_whole_step():
    m = KVCacheManager(full(), page_size=4, num_pages=5, max_requests=2)
    assert m.can_reserve_all([("a", 8), ("b", 12)])
    assert not m.can_reserve_all([("a", 9), ("b", 12)])
    assert m.reserve("a", 8)
    assert m.can_reserve_all([("a", 12), ("b", 8)]) and not m.can_reserve_all([("a", 12), ("b", 9)])
    assert m.reserve("b", 1)
    assert not m.can_reserve_all([("c", 1)])                             # no third state slot
    assert not m.reserve("c", 1)
    m.check()


def test_reserve_all_is_all_or_nothing_and_equals_single_reservations():
    a = KVCacheManager(full(), page_size=4, num_pages=6, max_requests=3)
    b = KVCacheManager(full(), page_size=4, num_pages=6, max_requests=3)
    assert a.reserve_all([("x", 5), ("y", 9)]) and b.reserve("x", 5) and b.reserve("y", 9)
    assert a.block_table(0, "x") == b.block_table(0, "x") and a.block_table(0, "y") == b.block_table(0, "y")
    before = (a.free_pages(), a.block_table(0, "x")[:], a.slots.num_free)
    assert not a.reserve_all([("x", 8), ("y", 12), ("z", 5)])           # one page short: nobody gets anything
    assert (a.free_pages(), a.block_table(0, "x"), a.slots.num_free) == before and "z" not in a.live_requests()
    assert a.reserve_all([("x", 8), ("y", 12)]) and a.free_pages() == 1   # x already has its 2 pages, y takes 1 more
    assert a.reserve_all([("x", 8), ("y", 12)]) and a.free_pages() == 1   # nothing new to take: a decode step inside a page
    with pytest.raises(CacheError):
        a.reserve_all([("x", 3)])                                         # a request does not shrink
    assert not a.reserve_all([("p", 1), ("q", 1)])                        # one state slot left, two newcomers
    a.check()


def test_groups_by_need_have_pages_of_their_own():
    needs = {0: CacheNeed(kv=KVNeed(2, 16)), 1: CacheNeed(kv=KVNeed(2, 16, window=8)),
             2: CacheNeed(kv=KVNeed(2, 16)), 3: CacheNeed(kv=KVNeed(1, 32)),
             4: CacheNeed(state=StateNeed((3, 5)))}
    m = KVCacheManager(needs, page_size=4, num_pages=6, max_requests=3)
    assert [g.cache_ids for g in m.groups] == [[0, 2], [1], [3]]
    assert m.reserve("a", 10)
    assert [m.block_table(g, "a") for g in range(3)] == [[0, 1, 2]] * 3   # each group counts from its own 0
    # the window group gives back what a query at position 10 cannot reach: keys before 3 -> no whole page yet
    assert m.release_passed("a", 10) == 0
    assert m.reserve("a", 14) and m.release_passed("a", 14) == 1          # first key needed 7 -> page 0 goes
    assert m.block_table(1, "a") == [-1, 1, 2, 3] and m.block_table(0, "a") == [0, 1, 2, 3]
    assert m.groups[1].pages.num_free == 3 and m.groups[0].pages.num_free == 2
    assert m.reserve("a", 24) and m.release_passed("a", 24) == 3          # first key needed 17 -> pages 1..3 go
    assert m.block_table(1, "a") == [-1, -1, -1, -1, 0, 4]                # page 0 came back and was used again first
    m.check()
    m.release("a")
    assert all(g.pages.num_free == 6 for g in m.groups)
    m.check()


def test_state_slots_follow_requests():
    slots = StateSlots(2)
    assert slots.take("a") == 0 and slots.take("b") == 1
    with pytest.raises(OutOfPages):
        slots.take("c")
    with pytest.raises(CacheError):
        slots.take("a")
    assert slots.give_back("a") == 0 and slots.take("c") == 0
    with pytest.raises(CacheError):
        slots.give_back("a")
    # the manager hands a slot to every request even when no cache holds state
    m = KVCacheManager(full(), page_size=4, num_pages=8, max_requests=2)
    assert m.reserve("x", 1) and m.reserve("y", 1) and {m.state_slot("x"), m.state_slot("y")} == {0, 1}
    m.release("x")
    assert m.reserve("z", 1) and m.state_slot("z") == 0
    assert not m.state                                                   # nothing to allocate for this model


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    window = rng.choice([None, 6, 20])
    needs = {0: CacheNeed(kv=KVNeed(2, 16)), 1: CacheNeed(kv=KVNeed(2, 16, window=window))}
    ps = rng.choice([1, 4, 16])
    m = KVCacheManager(needs, page_size=ps, num_pages=rng.randint(6, 20), max_requests=4, scatter_pages=seed % 2 == 1)
    live = {}
    next_id = 0
    for _ in range(600):
        op = rng.random()
        if op < 0.25 and len(live) < 6:
            rid, want = next_id, rng.randint(1, 3 * ps)
            next_id += 1
            before = [g.pages.num_free for g in m.groups]
            if m.reserve(rid, want):
                live[rid] = want
                m.release_passed(rid, want)
            else:
                assert [g.pages.num_free for g in m.groups] == before and not m.has(rid)
        elif op < 0.45 and live:
            # a whole step at once: some live requests grow, a newcomer may join; all or nothing
            step = {rid: live[rid] + rng.randint(0, ps + 1) for rid in rng.sample(list(live), rng.randint(1, len(live)))}
            if rng.random() < 0.3:
                step[next_id] = rng.randint(1, 2 * ps)
                next_id += 1
            before = ([g.pages.num_free for g in m.groups], {r: m.num_tokens(r) for r in live})
            if m.reserve_all(list(step.items())):
                for rid, want in step.items():
                    live[rid] = want
                    m.release_passed(rid, want)
            else:
                assert ([g.pages.num_free for g in m.groups], {r: m.num_tokens(r) for r in live}) == before
                assert all(m.has(r) == (r in live) for r in step)
        elif op < 0.75 and live:
            rid = rng.choice(list(live))
            want = live[rid] + rng.randint(1, 2 * ps)
            before = [list(m.block_table(g, rid)) for g in range(len(m.groups))]
            if m.reserve(rid, want):
                live[rid] = want
                m.release_passed(rid, want)
            else:
                assert [m.block_table(g, rid) for g in range(len(m.groups))] == before
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
        for rid, n in live.items():
            assert m.num_tokens(rid) == n
            for g in m.groups:
                table = g.tables[rid]
                assert len(table) == m.pages_for(n)
                first = g.first_needed_page(n)
                assert all(p >= 0 for p in table[first:])               # everything still readable is there
                if g.need.window is not None:
                    assert all(p == -1 for p in table[:first])           # everything passed has been given back
    for rid in list(live):
        m.release(rid)
    m.check()
    assert all(g.pages.num_free == g.pages.num_pages for g in m.groups) and m.slots.num_free == 4


def test_a_windowed_group_s_pool_is_sized_by_its_window_and_is_never_the_one_that_runs_out():
    """With a bound on the tokens one request brings to a step, the pool of a windowed group holds
    what ``max_requests`` windows and steps need, not the whole context: every request can then
    always take its step's pages there, however long it grows, if the pages the window has passed
    are given back after every step."""
    import random

    from nanoinfer_amd.parts.base import CacheNeed, KVNeed
    page, window, step_tokens, requests = 4, 10, 7, 3
    m = KVCacheManager({0: CacheNeed(kv=KVNeed(2, 16)), 1: CacheNeed(kv=KVNeed(2, 16, window=window))}, page, 400, requests,
                       max_step_tokens=step_tokens)
    full = next(g for g in m.groups if g.need.window is None)
    windowed = next(g for g in m.groups if g.need.window == window)
    assert full.pages.num_pages == 400
    assert windowed.pages.num_pages == requests * (-(-(window + step_tokens) // page) + 1) == 18
    assert m.max_tokens_per_request() == 400 * page
    rng = random.Random(3)
    held = {r: 0 for r in "abc"}
    for _ in range(600):
        r = rng.choice("abc")
        n = rng.randint(1, step_tokens)
        if held[r] + n > 120 * page // 3:          # stay inside the pool that keeps all keys
            m.release(r)
            held[r] = 0
            continue
        assert m.reserve(r, held[r] + n), "the windowed pool ran out"
        held[r] += n
        m.release_passed(r, held[r])
        m.check()
    # without the bound every group gets the whole pool
    m2 = KVCacheManager({0: CacheNeed(kv=KVNeed(2, 16, window=window))}, page, 400, requests)
    assert m2.groups[0].pages.num_pages == 400 and m2.max_tokens_per_request() == 1 << 60


def test_pages_that_a_byte_budget_buys():
    from nanoinfer_amd.parts.base import CacheNeed, KVNeed, StateNeed
    needs = {0: CacheNeed(kv=KVNeed(8, 64)), 1: CacheNeed(kv=KVNeed(8, 64)), 2: CacheNeed(state=StateNeed((4,)))}
    per_page = 2 * (2 * 8 * 16 * 64 * 2)            # two caches, keys and values, 16 tokens of 8 heads of 64 bfloat16
    assert KVCacheManager.pages_for_bytes(needs, 16, 10 * per_page + 5, torch.bfloat16) == 10
    assert KVCacheManager.pages_for_bytes(needs, 16, 10 * per_page, torch.float32) == 5
    assert KVCacheManager.pages_for_bytes({2: needs[2]}, 16, 1 << 30, torch.float32) == 0
    m = KVCacheManager(needs, 16, 10, 2, dtype=torch.bfloat16)
    assert m.pool_bytes() == 10 * per_page
