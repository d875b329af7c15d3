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
    return GroupSpec(entries=(0, 1), kv_heads=2, k_dim=16, v_dim=16, window=None, page_size=page_size)


def windowed(window, page_size=4):
    return GroupSpec(entries=(2,), kv_heads=2, k_dim=16, v_dim=16, window=window, page_size=page_size)


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


# ---- prefixes shared between requests ------------------------------------------------------------

def shared(pages=12, page_size=4, groups=1, max_requests=4):
    m = CacheManager([full(page_size)] * groups, [pages] * groups, max_requests=max_requests)
    m.enable_prefix_cache()
    return m


def run_whole(m, rid, tokens):
    m.add_request(rid)
    reused = m.adopt_prefix(rid, tokens)
    m.reserve(rid, len(tokens))
    m.commit(rid, len(tokens) - reused)
    m.remember_prefix(rid, tokens)
    return reused


def test_a_later_request_starts_behind_the_pages_it_shares():
    m = shared(groups=2)
    a = list(range(100, 111))                       # 11 tokens: two full pages and three tokens
    assert run_whole(m, "a", a) == 0
    assert m.cached_pages() == 2
    first_pages = [list(m.table("a", g)) for g in range(2)]
    m.free_request("a")
    m.check_invariants()
    assert m.pools[0].available == 10 and m.free_pages(0) == 12           # two pages stay, and count as room
    b = a[:8] + [7, 7, 7]
    assert run_whole(m, "b", b) == 8
    assert [m.table("b", g)[:2] for g in range(2)] == [t[:2] for t in first_pages]
    assert m.length("b") == 11 and m.prefix_hit_tokens == 8
    m.check_invariants()
    # the last token is always left to be computed: a prompt of exactly two known pages takes one
    m.add_request("c")
    assert m.adopt_prefix("c", a[:8]) == 4
    # a difference in the first page means nothing is shared, although the second page's tokens are the same
    m.add_request("d")
    assert m.adopt_prefix("d", [0] + a[1:]) == 0
    m.check_invariants()


def test_unused_prefixes_make_room_from_their_ends_and_oldest_first():
    m = shared(pages=6)
    old = list(range(0, 9))
    new = list(range(50, 59))
    run_whole(m, "old", old)
    m.free_request("old")
    run_whole(m, "new", new)
    m.free_request("new")
    assert m.cached_pages() == 4 and m.pools[0].available == 2 and m.free_pages(0) == 6
    m.add_request("x")
    m.reserve("x", 12)                              # three pages: one has to come from the older prefix, its second page
    m.check_invariants()
    assert m.cached_pages() == 3
    m.add_request("probe")
    assert m.adopt_prefix("probe", old) == 4        # the beginning of the older prefix is still there
    m.free_request("probe")
    m.add_request("y")
    m.reserve("y", 12)                              # all that is left
    m.check_invariants()
    assert m.cached_pages() == 0 and m.free_pages(0) == 0
    with pytest.raises(OutOfPages):
        m.reserve("y", 13)
    m.free_request("x")
    m.free_request("y")
    assert m.free_pages(0) == 6
    m.check_invariants()


def test_pages_in_use_are_never_given_up():
    m = shared(pages=4)
    a = list(range(9))
    run_whole(m, "a", a)                            # holds three pages, two of them known to the index
    m.add_request("b")
    assert m.adopt_prefix("b", a) == 8              # shares both
    assert m.free_pages(0) == 1
    assert not m.can_reserve("b", 17)
    m.free_request("a")                             # the pages stay held by b
    assert m.free_pages(0) == 2 and m.cached_pages() == 2
    m.reserve("b", 16)
    assert m.cached_pages() == 2
    m.check_invariants()


def test_two_requests_with_the_same_tokens_end_up_on_the_same_pages():
    m = shared(pages=8)
    tokens = list(range(10))
    for rid in ("a", "b"):                          # both admitted before either has computed anything
        m.add_request(rid)
        assert m.adopt_prefix(rid, tokens) == 0
        m.reserve(rid, 10)
    assert m.pools[0].available == 2
    m.commit("a", 10)
    m.remember_prefix("a", tokens)
    m.commit("b", 10)
    m.remember_prefix("b", tokens)                  # b's own two full pages go back
    assert m.table("a", 0)[:2] == m.table("b", 0)[:2] and m.table("a", 0)[2] != m.table("b", 0)[2]
    assert m.pools[0].available == 4
    m.check_invariants()
    m.free_request("a")
    m.free_request("b")
    assert m.free_pages(0) == 8 and m.clear_prefixes() == 2 and m.pools[0].available == 8
    m.check_invariants()


def test_tokens_that_are_not_final_are_not_entered():
    m = shared()
    tokens = list(range(7)) + [-1]
    m.add_request("a")
    m.reserve("a", 8)
    m.commit("a", 8)
    m.remember_prefix("a", tokens, known=7)
    assert m.cached_pages() == 1
    tokens[7] = 42
    m.remember_prefix("a", tokens, known=8)
    assert m.cached_pages() == 2
    m.check_invariants()


def test_windows_refuse_shared_prefixes():
    with pytest.raises(ValueError, match="keep all keys"):
        CacheManager([full(4), windowed(8, 4)], [8, 8], max_requests=2).enable_prefix_cache()
    with pytest.raises(ValueError, match="one page size"):
        CacheManager([full(4), full(8)], [8, 8], max_requests=2).enable_prefix_cache()


@pytest.mark.parametrize("seed", range(6))
def test_random_orders_with_shared_prefixes_keep_the_books(seed):
    """Requests draw their tokens from a few families with common beginnings; what a request adopts must hold exactly
    the tokens it asked for (each page remembers what was written to it)."""
    rng = random.Random(100 + seed)
    m = shared(pages=20, groups=2)
    families = [[rng.randrange(5) for _ in range(40)] for _ in range(3)]
    written = {}                                    # page of group 0 -> (position of its first token, its tokens)
    live, adopted, refused, next_id = {}, 0, 0, 0
    for _ in range(800):
        action = rng.random()
        if action < 0.3 and len(live) < 4:
            family = rng.choice(families)
            tokens = family[:rng.randrange(2, 40)]
            if rng.random() < 0.5:
                tokens = tokens[:-1] + [9]
            m.add_request(next_id)
            reused = m.adopt_prefix(next_id, tokens)
            for i in range(reused // 4):
                assert written[m.table(next_id, 0)[i]] == (i * 4, tokens[i * 4:i * 4 + 4])
            adopted += reused
            live[next_id] = [tokens, reused]
            next_id += 1
        elif action < 0.85 and live:
            rid = rng.choice(list(live))
            tokens, done = live[rid]
            if done == len(tokens):
                continue
            n = min(rng.choice([1, 2, 3, 5, 9]), len(tokens) - done)
            try:
                m.reserve(rid, done + n)
            except OutOfPages:
                refused += 1
                assert not m.can_reserve(rid, done + n)
            else:
                for pos in range(done, done + n):   # the step writes its tokens into the pages
                    page = m.table(rid, 0)[pos // 4]
                    if pos % 4 == 0:
                        written[page] = (pos, [])
                    assert written[page][0] == pos - pos % 4 and len(written[page][1]) == pos % 4
                    written[page][1].append(tokens[pos])
                m.commit(rid, n)
                live[rid][1] = done + n
                m.remember_prefix(rid, tokens, known=done + n)
                for i in range((done + n) // 4):    # a page taken from another request holds the same tokens
                    assert written[m.table(rid, 0)[i]] == (i * 4, tokens[i * 4:i * 4 + 4])
        elif live:
            rid = rng.choice(list(live))
            m.free_request(rid)
            del live[rid]
        m.check_invariants()
    for rid in list(live):
        m.free_request(rid)
    m.check_invariants()
    assert m.free_pages(0) == 20 and m.free_pages(1) == 20
    m.clear_prefixes()
    assert m.pools[0].available == 20 and m.pools[1].available == 20 and m.cached_pages() == 0
    assert adopted > 50 and refused > 0


def test_a_request_can_start_on_the_full_pages_of_another():
    m = CacheManager([full(4), full(4)], [10, 10], max_requests=3)
    m.add_request("first")
    m.reserve("first", 11)
    m.commit("first", 10)                           # two full pages and two tokens
    m.add_request("second")
    assert m.share_pages("first", "second", 9) == 8 and m.length("second") == 8
    assert [m.table("second", g) for g in range(2)] == [m.table("first", g)[:2] for g in range(2)]
    m.add_request("third")
    assert m.share_pages("first", "third", 7) == 4   # only pages wholly below the tokens that are the same
    m.reserve("second", 12)
    assert m.table("second", 0)[2] != m.table("first", 0)[2]
    m.check_invariants()
    assert m.share_pages("first", "second", 9) == 0  # only for a request that holds nothing
    m.free_request("first")
    m.check_invariants()
    assert m.free_pages(0) == 10 - 3                 # the shared pages stay with those who still hold them
    m.free_request("second")
    m.free_request("third")
    m.check_invariants()
    assert m.free_pages(0) == 10 and m.free_pages(1) == 10
    # where pages go back while a request runs, nothing is shared
    w = CacheManager([full(4), windowed(6, 4)], [10, 10], max_requests=2)
    w.add_request("a")
    w.reserve("a", 9)
    w.commit("a", 9)
    w.add_request("b")
    assert w.share_pages("a", "b", 8) == 0
