"""The cache manager's books (no GPU): no page is lost, held by more requests than the pool
counts, or freed twice, under random orders of requests (new ones, forks, steps, releases);
the window gives pages back; reservations and forks are all-or-nothing."""
import random

import pytest

from hf_cpu_amd.cache import CacheManager, OutOfPages, PagePool
from hf_cpu_amd.parts import FixedState, PagedKV
from hf_cpu_amd.status import EngineError


def manager(n_pages=8, page=4, slots=3, window=6, ctx=64):
    needs = [PagedKV(8, 8, 0), PagedKV(8, 8, window), PagedKV(8, 8, window), None, FixedState(5), PagedKV(8, 8, 0)]
    return CacheManager(needs, page, n_pages, slots, ctx)


def test_groups_follow_needs():
    m = manager()
    assert len(m.groups) == 2
    assert m.groups[0].entries == [0, 5] and m.groups[0].window == 0
    assert m.groups[1].entries == [1, 2] and m.groups[1].window == 6
    assert m.entry_group == [0, 1, 1, None, None, 0]
    assert m.state_entries == {4: 5}
    assert m.max_blocks == 16


def test_page_pool_refuses_double_free_and_overdraw():
    p = PagePool(3)
    a = p.take(2)
    with pytest.raises(OutOfPages):
        p.take(2)
    assert p.n_free == 1                     # all or nothing: the failed call took none
    p.give_back(a[:1])
    with pytest.raises(EngineError):
        p.give_back(a[:1])
    with pytest.raises(EngineError):
        p.give_back([7])
    p.check()
    p.give_back(a[1:])
    b = p.take(3)
    assert sorted(b) == [0, 1, 2] and p.reused == 2 and p.high_water == 3


def test_reserve_commit_release_and_window():
    m = manager(n_pages=8, page=4, window=6)
    h = m.admit("a")
    m.reserve("a", 10)                       # blocks 0..2 in both groups
    assert [len(t) for t in h.tables] == [3, 3]
    assert list(m.slot_rows("a", 0, 0, 10)) == [h.tables[0][p // 4] * 4 + p % 4 for p in range(10)]
    m.commit("a", 10)
    # next position 10, window 6: keys >= 5 stay visible, so block 0 (positions 0..3) goes
    assert h.tables[0] == [0, 1, 2] and h.tables[1][0] == -1 and h.tables[1][1:] == [1, 2]
    assert m.pools[1].n_held == 2 and m.pools[0].n_held == 3
    m.reserve("a", 1)
    m.commit("a", 1)                         # next position 11: keys >= 6, block 1 (4..7) still needed
    assert h.tables[1][1] == 1
    m.reserve("a", 2)
    m.commit("a", 2)                         # next position 13: keys >= 8, block 1 goes
    assert h.tables[1][:2] == [-1, -1] and m.pools[1].n_held == 2
    m.check()
    m.release("a")
    assert m.pools[0].n_held == m.pools[1].n_held == 0
    with pytest.raises(EngineError):
        m.release("a")
    m.check()


def test_no_block_table_entry_is_sent_twice_after_a_released_slot_is_taken_again():
    """A fork that ends before the next step leaves entries for its slot; the request that takes
    the slot next must not find them beside its own in one drain (a scatter has no order)."""
    m = manager(n_pages=8, page=4, slots=3)
    m.admit("a")
    m.reserve("a", 6)
    m.commit("a", 6)
    m.drain_appended(0), m.drain_appended(1)
    m.fork("a", "c")
    m.release("c")
    m.admit("y")
    m.reserve("y", 5)
    for g in range(2):
        sent = m.drain_appended(g)
        keys = [(slot, block) for slot, block, _ in sent]
        assert len(keys) == len(set(keys)), sent
        assert {(s_, b): p for s_, b, p in sent} == {(m.held["y"].slot, b): p for b, p in enumerate(m.held["y"].tables[g])}
    m.check()


def test_all_or_nothing_and_rollback():
    m = manager(n_pages=4, page=4)
    m.admit("a")
    m.admit("b")
    m.reserve("a", 9)                        # 3 pages
    with pytest.raises(OutOfPages):
        m.reserve("b", 5)                    # needs 2, one is free
    assert m.pools[0].n_free == 1 and m.held["b"].tables == [[], []]
    assert not m.can_reserve([("b", 5)]) and m.can_reserve([("b", 4)])
    assert m.pages_needed("c", 9) == [3, 3]  # a request not admitted yet
    m.rollback("a")                          # the step did not run
    assert m.pools[0].n_free == 4 and m.drain_appended(0) == []
    m.reserve("a", 3)
    m.commit("a", 3)
    m.reserve("a", 6)                        # positions 3..8: pages for blocks 1, 2
    m.rollback("a")
    assert len(m.held["a"].tables[0]) == 1 and m.held["a"].length == 3 and m.pools[0].n_held == 1
    with pytest.raises(EngineError) as e:
        m.reserve("a", 100)
    assert e.value.code == "ERANGE"
    m.admit("c")
    with pytest.raises(EngineError) as e:
        m.admit("d")
    assert e.value.code == "ENOMEM" and "slot" in str(e.value)
    m.check()


def test_appended_entries_reach_the_device_table_once():
    m = manager()
    h = m.admit("a")
    m.reserve("a", 5)
    app = m.drain_appended(0)
    assert app == [(h.slot, 0, h.tables[0][0]), (h.slot, 1, h.tables[0][1])]
    assert m.drain_appended(0) == []
    m.commit("a", 5)
    m.reserve("a", 2)                        # stays within block 1
    assert m.drain_appended(0) == []


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    m = manager(n_pages=12, page=4, slots=4, window=rng.choice([3, 6, 17]), ctx=40)
    live, counter = {}, 0
    for _ in range(600):
        r = rng.random()
        if (r < 0.25 and len(live) < 4) or not live:
            name = f"q{counter}"
            counter += 1
            if live and rng.random() < 0.4:    # start from another request's cache
                src = rng.choice(list(live))
                before = [p.n_free for p in m.pools]
                try:
                    copies, (s_from, s_to) = m.fork(src, name)
                except OutOfPages:
                    m.check()
                    assert name not in m.held and [p.n_free for p in m.pools] == before
                    continue
                live[name] = live[src]
                assert m.held[name].length == live[src] and s_from == m.held[src].slot and s_to == m.held[name].slot
                assert len(copies) == (len(m.groups) if live[src] % 4 else 0)
                for g, a, b in copies:         # the last, partly filled block: a page of its own
                    assert m.held[src].tables[g][live[src] // 4] == a and m.held[name].tables[g][live[src] // 4] == b != a
                for g in m.groups:             # whole blocks: the same pages
                    assert m.held[name].tables[g.index][:live[src] // 4] == m.held[src].tables[g.index][:live[src] // 4]
            else:
                m.admit(name)
                live[name] = 0
        elif r < 0.85:
            name = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 3, 5, 9, 14])
            try:
                m.reserve(name, n)
            except OutOfPages:
                before = [p.n_free for p in m.pools]
                m.check()
                assert [p.n_free for p in m.pools] == before
                continue
            except EngineError as e:
                assert e.code == "ERANGE" and live[name] + n > 40
                continue
            if rng.random() < 0.1:
                m.rollback(name)
            else:
                m.commit(name, n)
                live[name] += n
            h = m.held[name]
            assert h.length == live[name]
            for g in m.groups:                 # every position a later query can see has a page
                first = max(0, h.length - g.window + 1) if g.window else 0
                for pos in range(first, h.length):
                    assert h.tables[g.index][pos // 4] >= 0
        else:
            name = rng.choice(list(live))
            m.release(name)
            del live[name]
        m.check()
    for name in list(live):
        m.release(name)
    m.check()
    assert all(p.n_held == 0 for p in m.pools) and any(p.reused > 0 for p in m.pools)


def test_fork_shares_whole_pages_and_copies_the_last():
    m = manager(n_pages=8, page=4, slots=3, window=0, ctx=32)
    m.admit("a")
    m.reserve("a", 10)
    m.commit("a", 10)
    for g in range(len(m.groups)):
        m.drain_appended(g)
    copies, slots = m.fork("a", "b")
    a, b = m.held["a"], m.held["b"]
    assert b.length == 10 and slots == (a.slot, b.slot) and a.slot != b.slot
    for g in range(len(m.groups)):
        assert b.tables[g][:2] == a.tables[g][:2] and b.tables[g][2] != a.tables[g][2]
        assert (g, a.tables[g][2], b.tables[g][2]) in copies
        assert all(m.pools[g].holders(p) == 2 for p in a.tables[g][:2])
        assert sorted(m.drain_appended(g)) == sorted((b.slot, i, p) for i, p in enumerate(b.tables[g]))
        assert m.pools[g].n_held == 4                  # three of a's, one more for b
    m.check()
    # both go on independently; a shared page returns to the pool when its last holder lets go
    m.reserve("b", 3)
    m.commit("b", 3)
    m.reserve("a", 1)
    m.commit("a", 1)
    m.check()
    m.release("a")
    for g in range(len(m.groups)):
        assert m.pools[g].n_held == 4 and all(m.pools[g].holders(p) == 1 for p in b.tables[g])
    m.check()
    with pytest.raises(EngineError):                   # the name is taken
        m.fork("b", "b")
    m.truncate("b", 6)                                 # the page of position 6 is b's alone by now
    m.release("b")
    m.check()
    assert all(p.n_held == 0 for p in m.pools)


def test_fork_is_all_or_nothing_and_guards_shared_pages():
    m = manager(n_pages=3, page=4, slots=2, window=0, ctx=12)
    m.admit("a")
    m.reserve("a", 10)
    m.commit("a", 10)                                  # all three pages
    with pytest.raises(OutOfPages):
        m.fork("a", "b")                               # the copy of the last block needs a page
    assert "b" not in m.held and m.held["a"].length == 10
    m.check()
    m.truncate("a", 8)                                 # two whole pages: nothing to copy
    copies, _ = m.fork("a", "b")
    assert copies == [] and all(m.pools[g].n_held == 2 for g in range(len(m.groups)))
    with pytest.raises(EngineError) as e:              # a third request: no slot
        m.fork("a", "c")
    assert e.value.code == "ENOMEM"
    with pytest.raises(EngineError) as e:              # writing at position 6 would change b's keys too
        m.truncate("a", 6)
    assert e.value.code == "ENOTSUP"
    m.truncate("a", 4)                                 # a page boundary: a lets go of the second page, b keeps it
    m.check()
    m.reserve("a", 2)
    m.commit("a", 2)
    assert m.held["a"].tables[0][1] != m.held["b"].tables[0][1]
    m.check()
