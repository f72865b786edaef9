"""The cache manager: no page lost, held twice or freed twice, under random orders of requests."""
import random

import pytest

from leone_amd.cache.manager import CacheError, CacheManager, GroupSpec, OutOfPages, OutOfSlots


def test_reserve_commit_release_and_reuse():
    m = CacheManager([GroupSpec(4, 16)], max_requests=2, max_context=64)
    m.admit("a")
    m.reserve("a", 17)
    assert len(m.table("a", 0)) == 2
    first_pages = list(m.table("a", 0))
    m.commit("a")
    assert m.length("a") == 17 and m.free_pages(0) == 2
    m.reserve("a", 15)            # fills the second page exactly: no new page
    assert m.free_pages(0) == 2
    m.commit("a")
    m.reserve("a", 1)             # crosses into a third page
    assert m.free_pages(0) == 1
    m.commit("a")
    m.release("a")
    assert m.free_pages(0) == 4 and m.free_slots() == 2
    m.admit("b")
    m.reserve("b", 1)
    assert m.table("b", 0)[0] in first_pages + [3 - sum(first_pages) % 4, 0, 1, 2, 3]
    m.check()


def test_a_freed_page_is_the_next_one_used():
    m = CacheManager([GroupSpec(3, 8)], 3, 64)
    m.admit("a"); m.reserve("a", 8); m.commit("a")
    page = m.table("a", 0)[0]
    m.release("a")
    m.admit("b"); m.reserve("b", 3)
    assert m.table("b", 0) == [page]


def test_failed_reservation_changes_nothing_at_every_cut():
    # the reference rolls a failed allocation back at every cut point (crates/leone/src/kv.rs:1451-1473)
    for second_group_pages in range(0, 4):
        m = CacheManager([GroupSpec(8, 4), GroupSpec(max(1, second_group_pages), 4)], 2, 64)
        m.admit("a")
        before = (m.free_pages(0), m.free_pages(1), list(m.table("a", 0)), list(m.table("a", 1)))
        if second_group_pages < 4:
            with pytest.raises(OutOfPages) as error:
                m.reserve("a", 16)
            assert error.value.group == 1
            assert before == (m.free_pages(0), m.free_pages(1), list(m.table("a", 0)), list(m.table("a", 1)))
            m.check()


def test_rollback_is_exact():
    m = CacheManager([GroupSpec(6, 4)], 2, 64)
    m.admit("a"); m.reserve("a", 6); m.commit("a")
    snapshot = (list(m.table("a", 0)), m.free_pages(0), m.length("a"))
    m.reserve("a", 9)
    assert m.free_pages(0) < snapshot[1]
    m.rollback("a")
    assert snapshot == (list(m.table("a", 0)), m.free_pages(0), m.length("a"))
    m.reserve("a", 2); m.commit("a")
    assert m.length("a") == 8
    m.check()


def test_contract_violations():
    m = CacheManager([GroupSpec(4, 4)], 1, 10)
    with pytest.raises(CacheError):
        m.reserve("ghost", 1)
    m.admit("a")
    with pytest.raises(CacheError):
        m.admit("a")
    with pytest.raises(OutOfSlots):
        m.admit("b")
    with pytest.raises(CacheError):
        m.commit("a")                       # nothing reserved
    m.reserve("a", 3)
    with pytest.raises(CacheError):
        m.reserve("a", 1)                   # one transaction at a time
    with pytest.raises(CacheError):
        m.commit("a", 2)                    # not what was reserved
    m.commit("a", 3)
    with pytest.raises(CacheError):
        m.reserve("a", 8)                   # beyond the context of 10
    m.release("a")
    with pytest.raises(CacheError):
        m.release("a")                      # freed twice
    m.check()


def test_window_group_gives_pages_back_as_the_window_passes():
    m = CacheManager([GroupSpec(32, 4), GroupSpec(5, 4, window=6)], 1, 128)
    m.admit("a")
    m.reserve("a", 10); m.commit("a")
    # next query at 10 reads keys >= 5: block 0 (positions 0..3) is out of reach, block 1 (4..7) is not
    assert m.table("a", 1)[0] == -1 and m.table("a", 1)[1] >= 0
    assert m.table("a", 0)[0] >= 0            # the full group keeps everything
    for _ in range(100):
        m.reserve("a", 1); m.commit("a"); m.check()
        assert 5 - m.free_pages(1) <= 3        # never more than ceil((6-1)/4)+1 pages
    m.release("a")
    assert m.free_pages(1) == 5 and m.free_pages(0) == 32


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_every_page_accounted_for(seed):
    rng = random.Random(seed)
    groups = [GroupSpec(24, 8), GroupSpec(12, 8, window=rng.choice([5, 16, 23]))]
    m = CacheManager(groups, max_requests=4, max_context=96)
    live, names = {}, iter(range(10**6))
    for _ in range(1500):
        action = rng.random()
        if action < 0.15 and len(live) < 4:
            rid = next(names)
            m.admit(rid)
            live[rid] = 0
        elif action < 0.75 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 8, 9, 20])
            if live[rid] + n > 96:
                continue
            try:
                m.reserve(rid, n)
            except OutOfPages:
                m.check()
                continue
            if rng.random() < 0.15:
                m.rollback(rid)
            else:
                m.commit(rid)
                live[rid] += n
            assert m.length(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.release(rid)
            del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages(0) == 24 and m.free_pages(1) == 12 and m.free_slots() == 4


def test_fork_shares_full_pages_and_appends_go_to_private_ones():
    # fork shares storage, appends go to a private tail (crates/leone/src/kv.rs:1238-1274)
    m = CacheManager([GroupSpec(10, 4)], max_requests=3, max_context=64)
    m.admit("a"); m.reserve("a", 10); m.commit("a")                 # pages for blocks 0, 1, 2 (the last half full)
    shared = m.fork("a", "b")
    assert shared == 8 and m.length("b") == 8                        # rounded down to a page boundary
    assert m.table("b", 0) == m.table("a", 0)[:2] and m.shared_pages(0) == 2
    assert m.free_pages(0) == 7                                      # sharing took no page
    m.reserve("b", 3); m.commit("b")                                 # b's own tokens 8..10 go to a page of its own
    assert m.table("b", 0)[2] != m.table("a", 0)[2] and m.free_pages(0) == 6
    m.reserve("a", 5); m.commit("a")                                 # a goes on in its own tail
    assert m.table("a", 0)[:2] == m.table("b", 0)[:2]
    m.check()
    m.release("a")                                                   # shared pages stay while b holds them
    assert m.free_pages(0) == 10 - 3 and m.shared_pages(0) == 0
    m.check()
    m.release("b")
    assert m.free_pages(0) == 10
    m.check()
    # a fork of fewer tokens, and a fork of a fork
    m.admit("p"); m.reserve("p", 16); m.commit("p")
    assert m.fork("p", "q", tokens=9) == 8 and m.fork("q", "r") == 8
    assert m.holders(0, m.table("p", 0)[0]) == 3 and m.holders(0, m.table("p", 0)[2]) == 1
    with pytest.raises(CacheError):
        m.fork("p", "q")                                             # already admitted
    with pytest.raises(OutOfSlots):
        m.fork("p", "s")
    m.check()


def test_truncate_keeps_the_shared_prefix():
    # crates/leone/src/kv.rs:1276
    m = CacheManager([GroupSpec(10, 4)], 2, 64)
    m.admit("a"); m.reserve("a", 14); m.commit("a")
    m.fork("a", "b")                                                 # shares 12 tokens, 3 pages
    m.truncate("a", 13)                                              # inside a's private page: fine
    assert m.length("a") == 13 and len(m.table("a", 0)) == 4
    with pytest.raises(CacheError):
        m.truncate("a", 10)                                          # the page holding 10 is shared
    m.truncate("a", 8)                                               # a page boundary: a lets go of block 2, b keeps it
    assert m.table("a", 0) == m.table("b", 0)[:2] and m.holders(0, m.table("b", 0)[2]) == 1
    m.reserve("a", 2); m.commit("a")                                 # and writes on in a fresh page
    assert m.table("a", 0)[2] != m.table("b", 0)[2]
    with pytest.raises(CacheError):
        m.truncate("a", 11)
    m.check()
    m.release("a"); m.release("b"); m.check()
    assert m.free_pages(0) == 10


def test_fork_from_a_windowed_group_needs_the_pages_in_reach():
    m = CacheManager([GroupSpec(20, 4), GroupSpec(6, 4, window=6)], 3, 128)
    m.admit("a"); m.reserve("a", 20); m.commit("a")                  # window group has dropped blocks 0..2
    assert m.fork("a", "b") == 20 and m.table("b", 1)[:3] == [-1, -1, -1] and m.table("b", 1)[3] >= 0
    with pytest.raises(CacheError):
        m.fork("a", "c", tokens=8)                                   # keys 3..7 have left a's window
    m.check()


@pytest.mark.parametrize("seed", range(4))
def test_random_orders_with_forks(seed):
    rng = random.Random(50 + seed)
    m = CacheManager([GroupSpec(30, 4)], max_requests=5, max_context=80)
    live, names = {}, iter(range(10**6))
    for _ in range(1200):
        action = rng.random()
        if action < 0.12 and len(live) < 5:
            rid = next(names); m.admit(rid); live[rid] = 0
        elif action < 0.22 and live and len(live) < 5:
            parent = rng.choice(list(live)); rid = next(names)
            live[rid] = m.fork(parent, rid, rng.choice([None, live[parent] // 2]))
            assert live[rid] % 4 == 0 and live[rid] <= live[parent]
        elif action < 0.75 and live:
            rid = rng.choice(list(live)); n = rng.choice([1, 1, 2, 5, 9])
            if live[rid] + n > 80:
                continue
            try:
                m.reserve(rid, n)
            except OutOfPages:
                continue
            m.commit(rid); live[rid] += n
        elif action < 0.82 and live:
            rid = rng.choice(list(live))
            m.truncate(rid, live[rid] // 4 * 4 - (4 if live[rid] >= 4 and rng.random() < 0.5 else 0))
            live[rid] = m.length(rid)
        elif live:
            rid = rng.choice(list(live)); m.release(rid); del live[rid]
        m.check()
    for rid in list(live):
        m.release(rid)
    m.check()
    assert m.free_pages(0) == 30 and m.shared_pages(0) == 0


def test_the_log_of_freed_pages_names_every_page_whoever_frees_it():
    """With the log on, release, rollback, truncation and a window that has passed all leave their pages in
    it, once each; a shared page only when its last holder lets go; nothing while the log is off."""
    m = CacheManager([GroupSpec(12, 4), GroupSpec(12, 4, window=6)], max_requests=4, max_context=64)
    m.admit("a")
    m.reserve("a", 10)
    m.commit("a")
    m.release("a")
    assert m.drain_freed(0) == [] and m.drain_freed(1) == []           # off
    m.log_freed(True)
    m.admit("b")
    m.reserve("b", 9)
    table0 = [p for p in m.table("b", 0) if p >= 0]
    m.rollback("b")
    assert sorted(m.drain_freed(0)) == sorted(table0) and len(m.drain_freed(1)) == len(table0)
    m.reserve("b", 13)
    before = list(m.table("b", 1))
    m.commit("b")                                                       # the window of 6 has passed the first pages
    after = m.table("b", 1)
    passed = [p for b, p in enumerate(before) if p >= 0 and after[b] < 0]
    assert passed and sorted(m.drain_freed(1)) == sorted(passed) and m.drain_freed(0) == []
    m.release("b")
    m.check()
    assert m.free_pages(0) == 12 and m.free_pages(1) == 12
    # a shared page is named only when its last holder lets go
    m = CacheManager([GroupSpec(12, 4)], max_requests=4, max_context=64)
    m.log_freed(True)
    m.admit("b")
    m.reserve("b", 13)
    m.commit("b")
    m.fork("b", "c", 8)
    shared = [p for p in m.table("c", 0) if p >= 0]
    held = [p for p in m.table("b", 0) if p >= 0]
    assert len(shared) == 2
    m.release("b")
    assert sorted(m.drain_freed(0)) == sorted(set(held) - set(shared))     # the child still holds the shared ones
    m.release("c")
    assert sorted(m.drain_freed(0)) == sorted(shared)
    assert m.drain_freed(0) == []                                          # drained
    m.check()
    # a caller with too little room is refused and loses nothing: the pages come out when it asks again
    from ctypes import c_int
    m.admit("d")
    m.reserve("d", 13)
    held = sorted(p for p in m.table("d", 0) if p >= 0)
    m.release("d")
    small = (c_int * 2)()
    assert m._lib.leone_cache_drain_freed(m.handle, 0, small, 2) < 0
    assert sorted(m.drain_freed(0)) == held
