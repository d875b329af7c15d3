"""Cache manager: pages and slots are never lost, held twice or freed twice, under random orders
of requests; windows give pages back; a failed reservation changes nothing."""
import random

import pytest

from fllm_amd.cache import CacheManager, GroupSpec, OutOfPages, PagePool


def test_pool_is_lifo_and_counts_references():
    """rust/engine/src/mem/block_allocator.rs:383-392."""
    pool = PagePool(3)
    a, b = pool.alloc(), pool.alloc()
    assert (a, b) == (0, 1) and pool.available == 1
    pool.retain(a)
    assert pool.release(a) is False and pool.available == 1
    assert pool.release(a) is True and pool.available == 2
    assert pool.alloc() == a                      # last freed, first reused
    with pytest.raises(ValueError):
        pool.release(2)                           # never handed out
    pool.release(b)
    with pytest.raises(ValueError):
        pool.release(b)                           # freed twice
    with pytest.raises(ValueError):
        pool.retain(b)
    with pytest.raises(ValueError):
        pool.release(7)
    pool.alloc(), pool.alloc()
    with pytest.raises(OutOfPages):
        pool.alloc()


def full(page_size=4):
    return GroupSpec(entries=(0, 1), kv_heads=2, head_dim=16, window=None, page_size=page_size)


def windowed(window, page_size=4):
    return GroupSpec(entries=(2,), kv_heads=2, head_dim=16, window=window, page_size=page_size)


def test_reserve_commit_free():
    m = CacheManager([full()], [6], max_requests=2)
    assert m.add_request("a") == 0
    m.reserve("a", 9)
    assert m.table("a", 0) == [0, 1, 2] and m.free_pages() == 3
    m.commit("a", 9)
    assert m.length("a") == 9
    m.reserve("a", 10)                              # still inside the third page
    assert m.free_pages() == 3
    m.reserve("a", 13)
    assert m.table("a", 0) == [0, 1, 2, 3]
    m.check_invariants()
    m.free_request("a")
    assert m.free_pages() == 6 and m.free_slots() == 2
    m.free_request("a")                             # unknown request: nothing happens
    m.check_invariants()


def test_failed_reservation_changes_nothing():
    """rust/engine/src/mem/block_allocator.rs:394-409."""
    m = CacheManager([full(), windowed(8)], [4, 2], max_requests=2)
    m.add_request("a")
    m.reserve("a", 5)
    before = ([list(m.table("a", g)) for g in range(2)], [m.free_pages(g) for g in range(2)])
    assert not m.can_reserve("a", 13)               # the second group has no page left for it
    with pytest.raises(OutOfPages):
        m.reserve("a", 13)
    assert ([list(m.table("a", g)) for g in range(2)], [m.free_pages(g) for g in range(2)]) == before
    m.check_invariants()


def test_window_gives_pages_back():
    m = CacheManager([full(), windowed(6)], [16, 16], max_requests=1)
    m.add_request("a")
    held = []
    for step in range(40):
        m.reserve("a", m.length("a") + 1)
        m.commit("a", 1)
        n = m.length("a")
        table = m.table("a", 1)
        first_needed = max(0, n - 6 + 1) // 4
        assert all(p == -1 for p in table[:first_needed]) and all(p >= 0 for p in table[first_needed:])
        held.append(sum(p >= 0 for p in table))
        assert len(m.table("a", 0)) == -(-n // 4) and all(p >= 0 for p in m.table("a", 0))
        m.check_invariants()
    assert max(held) <= 3                           # a window of 6 over pages of 4 touches at most 3 pages
    assert m.free_pages(1) >= 13


def test_window_portion_keeps_what_its_first_row_sees():
    m = CacheManager([windowed(6)], [16], max_requests=1)
    m.add_request("a")
    m.reserve("a", 21)
    m.commit("a", 21)                               # next row at 21 sees 16..21
    assert [p >= 0 for p in m.table("a", 0)] == [False, False, False, False, True, True]
    m.reserve("a", 33)                              # a portion of 12 rows: its first row still needs page 4
    assert [p >= 0 for p in m.table("a", 0)] == [False] * 4 + [True] * 5
    m.commit("a", 12)
    assert [p >= 0 for p in m.table("a", 0)] == [False] * 7 + [True] * 2


def test_slots_and_duplicates():
    m = CacheManager([full()], [4], max_requests=2)
    assert {m.add_request("a"), m.add_request("b")} == {0, 1}
    with pytest.raises(ValueError):
        m.add_request("a")
    with pytest.raises(OutOfPages):
        m.add_request("c")
    m.free_request("a")
    assert m.add_request("c") == m.slot("c")
    with pytest.raises(KeyError):
        m.length("a")
    with pytest.raises(ValueError):
        m.commit("c", 1)                            # commits more than it holds pages for


def test_trim_returns_an_unused_reservation():
    m = CacheManager([full()], [8], max_requests=1)
    m.add_request("a")
    m.reserve("a", 30)
    m.commit("a", 5)
    m.trim("a", 6)
    assert len(m.table("a", 0)) == 2 and m.free_pages() == 6
    with pytest.raises(ValueError):
        m.trim("a", 4)


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_keep_the_books(seed):
    rng = random.Random(seed)
    groups = [full(4), windowed(rng.choice([3, 8, 17]), 4)]
    m = CacheManager(groups, [24, 24], max_requests=4)
    live, finished, refused = {}, 0, 0
    next_id = 0
    for _ in range(600):
        action = rng.random()
        if action < 0.25 and len(live) < 4:
            m.add_request(next_id)
            live[next_id] = 0
            next_id += 1
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 2, 5, 9, 20])
            try:
                m.reserve(rid, live[rid] + n)
            except OutOfPages:
                refused += 1
                assert not m.can_reserve(rid, live[rid] + n)
            else:
                m.commit(rid, n)
                live[rid] += n
                assert m.length(rid) == live[rid]
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
            finished += 1
        m.check_invariants()
    for rid in list(live):
        m.free_request(rid)
    m.check_invariants()
    assert m.free_pages(0) == 24 and m.free_pages(1) == 24 and m.free_slots() == 4
    assert finished > 10 and refused > 0


def test_window_group_looks_no_further_ahead_than_a_step():
    """With a bound on the tokens a step brings, a group that keeps a window holds pages for the window and one step,
    however long the prompt that a reservation covers; a pool made for that bound never runs dry, under random steps."""
    window, page, step = 10, 4, 7
    bound = CacheManager.window_pages_bound(window, page, step)
    assert bound == 5                                  # 9 keys behind the first row + 7 rows = 16 positions, + one edge
    requests = 3
    m = CacheManager([full(page), windowed(window, page)], [200, requests * bound], max_requests=requests, max_step_tokens=step)
    m.add_request("a")
    assert m.pages_missing("a", 101) == [26, 2]        # admission: the whole prompt in the full group, one step in the other
    m.reserve("a", 101)
    assert len([p for p in m.table("a", 1) if p >= 0]) == 2
    rng = random.Random(3)
    names = ["a", "b", "c"]
    m.add_request("b"), m.add_request("c")
    most = 0
    for _ in range(400):
        name = rng.choice(names)
        n = rng.randint(1, step)
        m.reserve(name, m.length(name) + n)
        most = max(most, max(sum(p >= 0 for p in m.table(x, 1)) for x in names))
        m.commit(name, n)
        m.check_invariants()
        if m.length(name) > 150:
            m.free_request(name)
            m.add_request(name)
    assert most == bound                               # the bound is reached, and never passed
    with pytest.raises(ValueError):
        m.commit("a", step + 40)                       # more than was reserved: a step longer than the bound
