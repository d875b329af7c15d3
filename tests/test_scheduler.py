"""The scheduler's decisions: admission, portions under the token budget, decode rows, what
happens when pages run out."""
import pytest

from fllm_amd.cache import CacheManager, GroupSpec
from fllm_amd.engine.scheduler import Scheduler, SchedulerConfig, Sequence
from fllm_amd.sampling import SamplingParams


def make(pages, max_seqs=4, budget=8, page_size=4, **kw):
    cache = CacheManager([GroupSpec(entries=(0,), kv_heads=1, k_dim=16, v_dim=16, window=None, page_size=page_size)], [pages],
                         max_requests=max_seqs)
    return Scheduler(SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=budget, **kw), cache, max_model_len=64), cache


def seq(sid, prompt_len, max_tokens=4):
    return Sequence(seq_id=sid, req_id=f"r{sid}", tokens=list(range(prompt_len)), prompt_len=prompt_len,
                    sampling=SamplingParams(max_tokens=max_tokens))


def run_step(s, cache, plan, new_token=1):
    """What the engine does after the forward pass."""
    for sid, start, count in plan.prefill:
        cache.commit(sid, count)
        s.commit_chunk(sid, count)
        q = s.sequences[sid]
        if q.num_computed == q.prefill_target:
            q.tokens.append(new_token)
            s.commit_decode(sid)
    for sid in plan.decode:
        cache.commit(sid, 1)
        s.sequences[sid].tokens.append(new_token)
        s.commit_decode(sid)


def test_prompt_is_cut_under_the_budget():
    s, cache = make(pages=16, budget=8)
    s.add(seq(0, 19))
    plans = []
    for _ in range(3):
        plan = s.schedule()
        plans.append(plan.prefill)
        run_step(s, cache, plan)
    assert plans == [[(0, 0, 8)], [(0, 8, 8)], [(0, 16, 3)]]
    plan = s.schedule()
    assert plan.prefill == [] and plan.decode == [0]


def test_decode_first_keeps_a_token_per_decoder():
    """rust/engine/src/scheduler.rs:1381-1397: budget 8 and two decoders leave 6 for the prompt."""
    for decode_first, expect in ((True, 6), (False, 8)):
        s, cache = make(pages=32, budget=8, decode_first=decode_first)
        s.add(seq(0, 3))
        s.add(seq(1, 3))
        run_step(s, cache, s.schedule())
        s.add(seq(2, 20))
        plan = s.schedule()
        assert plan.prefill == [(2, 0, expect)]
        assert plan.decode == ([0, 1] if decode_first else [])       # without it the prompt eats the budget


def test_admission_reserves_prompt_plus_one_and_is_first_come_first_served():
    s, cache = make(pages=4, budget=64)                 # 16 tokens of cache
    s.add(seq(0, 12))                                   # needs 13 tokens: 4 pages
    s.add(seq(1, 2))                                    # would fit, but waits behind nobody: the pool is full
    plan = s.schedule()
    assert [p[0] for p in plan.prefill] == [0] and list(s.waiting) == [1]
    assert cache.free_pages() == 0
    s2, cache2 = make(pages=4, budget=64)
    s2.add(seq(0, 40))                                  # never fits: blocks the queue (head of line)
    s2.add(seq(1, 2))
    assert s2.schedule() is None and list(s2.waiting) == [0, 1]


def test_watermark_only_counts_when_others_run():
    """rust/engine/src/scheduler.rs:1365-1378."""
    s, cache = make(pages=4, budget=64, watermark_pages=2)
    s.add(seq(0, 6))                                    # 2 pages; nothing runs, so no watermark
    plan = s.schedule()
    assert [p[0] for p in plan.prefill] == [0]
    run_step(s, cache, plan)
    s.add(seq(1, 3))                                    # 1 page + watermark 2 > 2 free
    s.schedule()
    assert list(s.waiting) == [1]


def test_max_num_seqs():
    s, cache = make(pages=32, max_seqs=2, budget=64)
    for i in range(3):
        s.add(seq(i, 3))
    s.schedule()
    assert s.running == [0, 1] and list(s.waiting) == [2]


def test_partial_prefill_limits():
    """rust/engine/src/scheduler.rs:1400-1415."""
    s, cache = make(pages=64, budget=12, max_partial_prefills=2)
    for i in range(3):
        s.add(seq(i, 5))
    assert [p[0] for p in s.schedule().prefill] == [0, 1]
    s, cache = make(pages=64, budget=64, long_prefill_threshold=8, max_long_partial_prefills=1)
    s.add(seq(0, 20))
    s.add(seq(1, 20))
    s.add(seq(2, 4))
    assert [p[0] for p in s.schedule().prefill] == [0, 2]   # the second long prompt waits, the short one goes


def test_pages_run_out_newest_sequence_is_preempted_and_recomputed():
    """rust/engine/src/scheduler.rs:933-968, :647-657, :1332."""
    s, cache = make(pages=4, budget=64, page_size=4)
    s.add(seq(0, 6, max_tokens=8))                      # 7 tokens reserved: 2 pages
    s.add(seq(1, 6, max_tokens=8))                      # 2 pages
    run_step(s, cache, s.schedule())                    # both prompts done, one token each: 7 tokens held
    for _ in range(2):                                  # positions 6 and 7 fit in the second page of each
        plan = s.schedule()
        assert plan.decode == [0, 1]
        run_step(s, cache, plan)
    plan = s.schedule()                                 # position 8 needs a third page for both: none left
    assert plan.decode == [0] and s.preemptions == 1
    assert list(s.waiting) == [1] and s.running == [0]
    victim = s.sequences[1]
    assert victim.num_computed == 0 and victim.prefill_target == len(victim.tokens) == 9 and victim.preempted
    assert not cache.has_request(1)
    run_step(s, cache, plan)
    for _ in range(20):                                 # 0 finishes, then 1 is admitted again and recomputed
        plan = s.schedule()
        if plan is None:
            break
        run_step(s, cache, plan)
        for sid in list(s.running):
            if s.sequences[sid].remaining() <= 0:
                s.finish(sid)
    assert not s.has_work() and cache.free_pages() == 4
    cache.check_invariants()


def test_a_single_sequence_is_never_preempted_for_itself():
    s, cache = make(pages=2, budget=64, page_size=4)
    s.add(seq(0, 7, max_tokens=8))                      # 8 tokens: both pages
    run_step(s, cache, s.schedule())
    run_step(s, cache, s.schedule())                    # the row at position 7 still fits
    assert s.schedule() is None                         # position 8 has no page; the engine reports no progress
    assert s.preemptions == 0 and s.running == [0]


def test_finish_gives_everything_back():
    s, cache = make(pages=8, budget=64)
    s.add(seq(0, 5))
    run_step(s, cache, s.schedule())
    s.finish(0)
    assert cache.free_pages() == 8 and not s.has_work() and cache.free_slots() == 4


def prioritized(sid, prompt_len, priority, max_tokens=8):
    return Sequence(seq_id=sid, req_id=f"r{sid}", tokens=list(range(prompt_len)), prompt_len=prompt_len,
                    sampling=SamplingParams(max_tokens=max_tokens, priority=priority))


def test_priority_policy_serves_the_smaller_value_first_and_fcfs_ignores_it():
    """rust/engine/src/scheduler.rs:1308-1319: two requests of priorities 5 and 1; first come, first served runs both in
    arrival order; with one slot under the priority policy the smaller value runs."""
    s, _ = make(pages=64, max_seqs=2, budget=16)
    s.add(prioritized(1, 4, 5))
    s.add(prioritized(2, 4, 1))
    s.schedule()
    assert s.running == [1, 2]
    s, _ = make(pages=64, max_seqs=1, budget=16, policy="priority")
    s.add(prioritized(1, 4, 5))
    s.add(prioritized(2, 4, 1))
    s.schedule()
    assert s.running == [2]


def test_a_better_priority_takes_the_slot_of_the_worst_running_sequence():
    """rust/engine/src/scheduler.rs:1322-1339: the preempted sequence waits again with nothing computed; an equal
    priority never preempts; first come, first served never preempts for a waiting request (:1341-1350)."""
    s, cache = make(pages=64, max_seqs=1, budget=16, policy="priority")
    s.add(prioritized(1, 4, 5))
    run_step(s, cache, s.schedule())
    assert s.running == [1]
    s.add(prioritized(2, 4, 0))
    plan = s.schedule()
    assert s.running == [2] and 1 in s.waiting and s.preemptions == 1
    assert s.sequences[1].num_computed == 0 and not cache.has_request(1)
    assert plan.prefill == [(2, 0, 4)]
    s.add(prioritized(3, 4, 0))
    s.schedule()
    assert s.running == [2] and s.preemptions == 1
    cache.check_invariants()
    s, cache = make(pages=64, max_seqs=1, budget=16)
    s.add(prioritized(1, 4, 9))
    s.schedule()
    s.add(prioritized(2, 4, -9))
    s.schedule()
    assert s.running == [1] and s.preemptions == 0


def test_a_full_pool_admits_by_priority_through_preemption():
    """rust/engine/src/scheduler.rs:1352-1363: 4 pages of 4 tokens; a 12-token prompt (3 pages and one for its first
    token) fills the pool, a better request gets its pages."""
    s, cache = make(pages=4, max_seqs=4, budget=16, policy="priority")
    s.add(prioritized(1, 12, 5))
    s.schedule()
    assert s.running == [1]
    s.add(prioritized(2, 12, 0))
    s.schedule()
    assert s.running == [2] and s.preemptions == 1
    cache.check_invariants()


def test_priority_orders_the_running_sequences_and_picks_the_worst_when_pages_run_out():
    """Running sequences are served in (priority, arrival) order, and a decode row that finds no page sends the
    sequence of the worst priority back to the queue, not the newest."""
    s, cache = make(pages=3, max_seqs=3, budget=16, policy="priority")
    s.add(prioritized(1, 3, 7))          # the worst priority, the oldest
    s.add(prioritized(2, 3, 0))
    s.add(prioritized(3, 3, 3))
    plan = s.schedule()
    assert [p[0] for p in plan.prefill] == [2, 3, 1]
    run_step(s, cache, plan)
    plan = s.schedule()
    assert plan.decode == [2, 3, 1]      # the fourth token of each still fits its one page
    run_step(s, cache, plan)
    # The fifth token needs a second page and none is free.  Request 2 is served first and takes the page of the worst
    # one (1, not the newest, 3); request 3 then finds no page either, and the only other sequence gives way to it,
    # better though it is: whoever needs a page takes it from the worst of the others (scheduler.rs:433-445, :646-658).
    plan = s.schedule()
    assert plan.decode == [3] and s.preemptions == 2 and s.running == [3] and set(s.waiting) == {1, 2}
    cache.check_invariants()


# ---- prefix cache --------------------------------------------------------------------------------

def test_a_request_starts_behind_the_prefix_the_cache_knows():
    s, cache = make(pages=16, budget=8, prefix_cache=True)
    s.add(seq(0, 11, max_tokens=1))
    while s.has_work():
        plan = s.schedule()
        run_step(s, cache, plan)
        for sid in [sid for sid, q in s.sequences.items() if q.remaining() <= 0]:
            s.finish(sid)
    assert cache.cached_pages() == 2 and cache.free_pages() == 16     # the keys of 11 tokens were computed: two full pages
    s.add(seq(1, 14))                               # the same first 11 tokens and three more
    plan = s.schedule()
    assert plan.prefill == [(1, 8, 6)]              # two pages are taken over
    assert cache.prefix_hit_tokens == 8
    run_step(s, cache, plan)
    cache.check_invariants()


def test_a_preempted_sequence_finds_its_pages_again():
    s, cache = make(pages=6, budget=16, prefix_cache=True)
    s.add(seq(0, 8, max_tokens=7))
    s.add(Sequence(seq_id=1, req_id="r1", tokens=list(range(100, 107)), prompt_len=7, sampling=SamplingParams(max_tokens=8)))
    run_step(s, cache, s.schedule())                # both prompts: 3 + 2 pages
    assert cache.free_pages() == 1
    for _ in range(4):
        run_step(s, cache, s.schedule())            # sequence 1 takes the last page with its ninth token
    assert cache.free_pages() == 0 and cache.cached_pages() == 5
    plan = s.schedule()                             # sequence 0 needs a fourth page: the newest gives way
    assert s.preemptions == 1 and s.sequences[1].state == "waiting" and plan.decode == [0]
    # sequence 1 had computed 11 tokens: its third page goes to sequence 0, its two full pages stay known
    assert cache.pools[0].available == 0 and cache.free_pages() == 2 and cache.cached_pages() == 5
    run_step(s, cache, plan)
    plan = s.schedule()
    assert plan.decode == [0] and not plan.prefill  # sequence 1 needs four pages: its own two and two more, which are not there
    assert cache.free_pages() == 2
    run_step(s, cache, plan)
    assert s.sequences[0].remaining() == 0
    s.finish(0)
    plan = s.schedule()
    assert plan.prefill == [(1, 8, 4)]              # it goes on behind its two pages
    run_step(s, cache, plan)
    cache.check_invariants()
    # without the room for them, the same pages are given up: another request takes everything
    s.finish(1)
    s.add(Sequence(seq_id=2, req_id="r2", tokens=list(range(200, 222)), prompt_len=22, sampling=SamplingParams(max_tokens=1)))
    plan = s.schedule()
    assert plan.prefill == [(2, 0, 16)] and cache.cached_pages() == 0 and cache.free_pages() == 0
    cache.check_invariants()


def test_a_blocked_request_leaves_the_prefix_index_as_it_was():
    """The request at the head of the queue is tried at every call while it does not fit: its hits are counted once, when
    it is admitted, and the pages it would take over keep their place among the unused ones."""
    s, cache = make(pages=8, budget=32, prefix_cache=True)
    for sid, first in ((0, 0), (1, 100)):           # two prompts of 9 tokens leave two known pages each
        s.add(Sequence(seq_id=sid, req_id=f"r{sid}", tokens=list(range(first, first + 9)), prompt_len=9,
                       sampling=SamplingParams(max_tokens=1)))
        while s.has_work():
            run_step(s, cache, s.schedule())
            for done in [d for d, q in s.sequences.items() if q.remaining() <= 0]:
                s.finish(done)
    assert cache.cached_pages() == 4 and cache.prefix_hit_tokens == 0
    order = list(cache._idle)
    s.add(Sequence(seq_id=2, req_id="r2", tokens=list(range(300, 320)), prompt_len=20, sampling=SamplingParams(max_tokens=12)))
    run_step(s, cache, s.schedule())                # 6 pages held: the unused prefixes of request 0 had to go
    assert cache.pools[0].available == 0 and cache.free_pages() == 2
    order = list(cache._idle)
    assert len(order) == 2
    # the first prompt of request 1 again, and more: it needs 2 known + 3 further pages, 2 + 0 are there
    s.add(Sequence(seq_id=3, req_id="r3", tokens=list(range(100, 117)), prompt_len=17, sampling=SamplingParams(max_tokens=1)))
    for _ in range(3):
        plan = s.schedule()
        assert plan.prefill == [] and plan.decode == [2] and 3 in s.waiting
        assert cache.prefix_hit_tokens == 0 and list(cache._idle) == order
        run_step(s, cache, plan)
    cache.check_invariants()
    s.finish(2)
    plan = s.schedule()
    assert plan.prefill == [(3, 8, 9)] and cache.prefix_hit_tokens == 8
    cache.check_invariants()


def test_portions_end_on_multiples_and_at_the_place_where_state_is_copied():
    """scheduler.rs:383-388: a portion ends exactly on the boundary that is worth keeping; and a model may ask for
    portions that begin on multiples of some number of tokens."""
    s, cache = make(pages=32, budget=10, page_size=4, portion_multiple=3)
    s.add(seq(0, 29))
    cuts = []
    while s.sequences[0].num_computed < 29:
        plan = s.schedule()
        cuts += plan.prefill
        run_step(s, cache, plan)
    assert cuts == [(0, 0, 9), (0, 9, 9), (0, 18, 9), (0, 27, 2)]          # multiples of 3 until the prompt ends
    s, cache = make(pages=32, budget=10, page_size=4, portion_multiple=3, state_checkpoints=True, prefix_cache=True)
    s.add(seq(0, 29))
    cuts, copied = [], []
    while s.sequences[0].num_computed < 29:
        plan = s.schedule()
        cuts += plan.prefill
        run_step(s, cache, plan)
        for sid, tokens in s.take_checkpoints():
            copied.append((sid, tokens, s.sequences[sid].num_computed))
            s.keep_checkpoint(sid, tokens, "copy of the state behind 24 tokens")
    # pages of 4 and multiples of 3: the state is copied behind 24 tokens, the last place below the last token that is both
    assert cuts == [(0, 0, 9), (0, 9, 9), (0, 18, 6), (0, 24, 5)] and copied == [(0, 24, 24)]
    s.finish(0)
    s.add(Sequence(seq_id=1, req_id="r1", tokens=list(range(26)) + [77, 78], prompt_len=28, sampling=SamplingParams(max_tokens=1)))
    plan = s.schedule()
    assert plan.prefill == [(1, 24, 4)] and s.take_restores() == [(1, "copy of the state behind 24 tokens")]
    # a prompt that shares fewer pages than the copy stands for starts from nothing: pages alone are not enough
    s.add(Sequence(seq_id=2, req_id="r2", tokens=list(range(20)) + [90] * 8, prompt_len=28, sampling=SamplingParams(max_tokens=1)))
    run_step(s, cache, plan)
    plan = s.schedule()
    assert (2, 0, 9) in plan.prefill and s.take_restores() == []
    cache.check_invariants()
