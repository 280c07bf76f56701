"""The cache manager's bookkeeping, without a GPU: the reference's literal vectors, and under random
orders of requests no page is lost, held twice or freed twice."""
import numpy as np
import pytest

from simply_amd.cache import CacheError, CacheManager, OutOfPages, PagePool
from simply_amd.parts.base import PagedKVNeed, StateNeed

GLOBAL = PagedKVNeed(1, 2, None)


def manager(needs, page_size, num_pages, slots=3, max_len=10000):
    return CacheManager([(n, None) for n in needs], page_size=page_size, num_pages=num_pages, num_slots=slots,
                        max_seq_len=max_len)


def tables(m, gid, rids):
    return [m.groups[gid].pages_of(r) for r in rids]


def test_allocate_vector():
    """simply/utils/ragged_paged_attention_test.py:83-106: 6 pages of 3 tokens, lengths [3, 0, 4]."""
    m = manager([GLOBAL], 3, 6)
    for r in "abc":
        m.admit(r)
    m.reserve("a", 0, 3)
    m.reserve("b", 0, 0)
    m.reserve("c", 0, 4)
    assert tables(m, 0, "abc") == [[0], [], [1, 2]]
    assert m.groups[0].pool.free_list() == [3, 4, 5]
    m.check()


def test_allocate_vector_after_reuse():
    """simply/utils/ragged_paged_attention_test.py:108-126: free list [5, 2, 4, 0], tables [[3], [1], []],
    lengths [3, 2, 0], then 5, 0 and 6 more tokens -> [[3, 5, 2], [1], [4, 0]] and nothing free."""
    m = manager([GLOBAL], 3, 6)
    g = m.groups[0]
    for r in "abc":
        m.admit(r)
    # bring the pool into the state of the vector: take all, give back in the order 5, 2, 4, 0
    g.pool.take(6)
    g.pool.give_back([5, 2, 4, 0])
    g.table[m.slot_of("a"), 0] = 3
    g.seqs["a"].num_tokens = 3
    g.table[m.slot_of("b"), 0] = 1
    g.seqs["b"].num_tokens = 2
    m.check()
    m.reserve("a", 3, 5)
    m.reserve("b", 2, 0)
    m.reserve("c", 0, 6)
    assert tables(m, 0, "abc") == [[3, 5, 2], [1], [4, 0]]
    assert g.pool.free_list() == []
    with pytest.raises(OutOfPages):
        m.reserve("b", 2, 2)
    m.check()


def test_release_for_window_vector():
    """simply/utils/ragged_paged_attention_test.py:501-525: 9 pages of 4, window_size 5 (6 keys visible with
    the query's own), lengths [3, 8, 10]: the third request gives back its first page."""
    m = manager([PagedKVNeed(1, 2, 6)], 4, 9)
    for r, n in zip("abc", (3, 8, 10)):
        m.admit(r)
        m.reserve(r, 0, n)
    assert tables(m, 0, "abc") == [[0], [1, 2], [3, 4, 5]]
    for r, n in zip("abc", (3, 8, 10)):
        m.reserve(r, n, 0)  # the release that precedes every allocation
    assert tables(m, 0, "abc") == [[0], [1, 2], [4, 5]]
    assert m.groups[0].pool.free_list() == [6, 7, 8, 3]
    # the table keeps absolute block numbers: block 0 of "c" is a hole now
    assert list(m.groups[0].table[m.slot_of("c"), :4]) == [-1, 4, 5, -1]
    m.check()


def test_groups_by_need_and_state_slots():
    needs = [PagedKVNeed(2, 16, 8), PagedKVNeed(2, 16, None), PagedKVNeed(2, 16, 8), StateNeed((3, 4)), None,
             PagedKVNeed(1, 16, None)]
    m = manager(needs, 4, 10)
    assert len(m.groups) == 3
    assert [v.group_id for v in m.views] == [0, 1, 0, None, None, 2]
    slots = [m.admit(r) for r in "abc"]
    assert sorted(slots) == [0, 1, 2]
    with pytest.raises(CacheError):
        m.admit("d")          # no slot left
    with pytest.raises(CacheError):
        m.admit("a")          # twice
    m.free("b")
    assert m.admit("d") == slots[1]
    m.check()


def test_cache_from_shares_storage():
    needs = [(PagedKVNeed(2, 16, None), None), (PagedKVNeed(2, 16, None), 0), (PagedKVNeed(2, 16, 4), None)]
    m = CacheManager(needs, page_size=4, num_pages=8, num_slots=2, max_seq_len=64)
    assert m.views[1].group_id == m.views[0].group_id and not m.views[1].write and m.views[0].write
    with pytest.raises(CacheError):
        CacheManager([(PagedKVNeed(2, 16, None), None), (PagedKVNeed(2, 16, 4), 0)], page_size=4, num_pages=8,
                     num_slots=2, max_seq_len=64)


def test_windowed_group_holds_a_window_only():
    W, P = 8, 4
    m = manager([PagedKVNeed(1, 2, W), GLOBAL], P, 100, slots=1)
    m.admit("r")
    n = 0
    for q in [3, 1, 1, 7, 2, 1, 1, 1, 20, 1, 1, 1, 1, 5, 1]:
        m.reserve("r", n, q)
        for gid in (0, 1):
            m.check_readable(gid, "r", n, q)
        n += q
        local = len(m.groups[0].pages_of("r"))
        # pages for the keys the first query of the portion sees up to the portion's end
        lo = max(n - q - W + 1, 0)
        assert local == -(-n // P) - lo // P
        assert len(m.groups[1].pages_of("r")) == -(-n // P)
    m.free("r")
    assert all(g.pool.num_free == 100 for g in m.groups)


def test_windowed_group_has_a_pool_of_its_own_size():
    """A windowed group's pool holds what its requests can hold at once (the reference sizes its local pool by the
    window: simply/utils/ragged_paged_attention.py:95-110, simply/serving/page_server.py:180-196), not what the
    group that keeps every key needs; and a long request still runs in it, portion by portion."""
    from simply_amd.cache.manager import windowed_pool_pages
    W, P, slots, step = 64, 16, 3, 128
    m = CacheManager([(PagedKVNeed(1, 2, W), None), (GLOBAL, None)], page_size=P, num_pages=3 * 512, num_slots=slots,
                     max_seq_len=8192, max_step_tokens=step)
    assert m.groups[1].pool.num_pages == 3 * 512
    assert m.groups[0].pool.num_pages == windowed_pool_pages(W, P, slots, step) == 3 * (4 + 2) + 8
    # the group that keeps every key could hold each of three requests of 8192 tokens; the windowed pool is tight
    rng = np.random.default_rng(0)
    done = {r: 0 for r in "abc"}
    for r in done:
        assert m.can_hold(8192, step)
        m.admit(r)
    most = 0
    while any(n < 8192 for n in done.values()):
        # a step: every request brings something, together at most `step` tokens, cut anywhere
        left = step
        wants = []
        for r in sorted(done, key=lambda _: rng.random()):
            q = min(int(rng.integers(1, 100)), left, 8192 - done[r])
            if q > 0:
                wants.append((r, done[r], q))
                left -= q
        m.reserve_all(wants)                      # never short of pages
        for r, start, q in wants:
            m.check_readable(0, r, start, q)
            done[r] += q
        for r in done:                            # a request that the step left out can go on where it stands
            m.check_readable(0, r, done[r], 0)
        m.mark_issued(wants)                      # the step has been handed to the GPU
        most = max(most, m.groups[0].pool.num_pages - m.groups[0].pool.num_free)
        m.check()
    assert most <= m.groups[0].pool.num_pages and most >= 3 * 4
    # a function may give a group another size
    m2 = CacheManager([(PagedKVNeed(1, 2, W), None), (GLOBAL, None)], page_size=P, num_pages=100, num_slots=2,
                      max_seq_len=512, group_pages=lambda need, pages: 7 if need.window else pages)
    assert [g.pool.num_pages for g in m2.groups] == [7, 100]


def test_a_steps_reservations_give_back_before_they_take():
    """Two requests in one step, no free page: the first needs two new pages, the second's window gives two back.
    Whichever comes first in the list, the step fits; and when it does not fit, nothing has changed."""
    W, P = 4, 2
    for order in (("a", "b"), ("b", "a")):
        m = manager([PagedKVNeed(1, 2, W)], P, 8, slots=2)
        m.admit("a")
        m.admit("b")
        m.reserve("a", 0, 4)           # a: blocks 0, 1
        m.reserve("b", 0, 12)          # b: all of its 12 tokens in one step, blocks 0..5
        assert m.groups[0].pool.num_free == 0
        wants = {"a": ("a", 4, 4), "b": ("b", 12, 1)}   # a: two new pages; b: blocks 0..3 are dead at position 12, one new
        assert m.can_reserve([wants[r] for r in order])
        m.reserve_all([wants[r] for r in order])
        m.check()
        assert len(m.groups[0].pages_of("a")) == 4 and len(m.groups[0].pages_of("b")) == 3
        assert m.groups[0].pool.num_free == 1
        # one more page than there is: refused, nothing changed
        before = m.groups[0].table.copy(), m.groups[0].pool.free_list()
        with pytest.raises(OutOfPages):
            m.reserve_all([("a", 8, 10), ("b", 13, 1)])     # five new pages, four to be had
        assert (before[0] == m.groups[0].table).all() and before[1] == m.groups[0].pool.free_list()


def test_errors():
    pool = PagePool(3)
    pages = pool.take(2)
    pool.give_back(pages)
    with pytest.raises(CacheError):
        pool.give_back([pages[0]])  # freed twice
    with pytest.raises(OutOfPages):
        pool.take(4)
    m = manager([GLOBAL], 4, 4, max_len=16)
    m.admit("a")
    with pytest.raises(CacheError):
        m.reserve("a", 0, 17)       # beyond max_seq_len
    m.reserve("a", 0, 9)
    m.admit("b")
    with pytest.raises(OutOfPages):
        m.reserve("b", 0, 5)        # two pages wanted, one free
    assert m.groups[0].pool.num_free == 1   # the refused reservation changed nothing
    with pytest.raises(KeyError):
        m.free("zzz")
    m.check()


@pytest.mark.parametrize("seed", range(8))
def test_random_orders_lose_nothing(seed):
    rng = np.random.default_rng(seed)
    P = int(rng.choice([1, 3, 4, 16]))
    num_pages = int(rng.integers(12, 40))
    needs = [PagedKVNeed(1, 2, int(rng.integers(1, 20))), GLOBAL, PagedKVNeed(1, 2, int(rng.integers(1, 20)))]
    m = manager(needs, P, num_pages, slots=4, max_len=num_pages * P)
    live, serial = {}, 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and m.has_slot():
            rid = f"r{serial}"
            serial += 1
            m.admit(rid)
            live[rid] = 0
        elif action < 0.85 and live:
            rid = str(rng.choice(sorted(live)))
            q = int(rng.integers(1, 12))
            if live[rid] + q > num_pages * P:
                continue
            before = [g.pool.num_free for g in m.groups], [g.pages_of(rid) for g in m.groups]
            if m.can_reserve([(rid, live[rid], q)]):
                m.reserve(rid, live[rid], q)
                for g in m.groups:
                    m.check_readable(g.group_id, rid, live[rid], q)
                    assert (m.slot_mapping(g.group_id, rid, live[rid], q) >= 0).all()
                live[rid] += q
            else:
                with pytest.raises(OutOfPages):
                    m.reserve(rid, live[rid], q)
                assert before == ([g.pool.num_free for g in m.groups], [g.pages_of(rid) for g in m.groups])
        elif live:
            rid = str(rng.choice(sorted(live)))
            m.free(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.free(rid)
    m.check()
    assert all(g.pool.num_free == num_pages for g in m.groups)
