"""Continuous-batching scheduler: admits requests, cuts prompts into portions under a token
budget, schedules one decode token per running sequence, and decides what happens when pages
run out.  Behaviour follows the reference's scheduler (rust/engine/src/scheduler.rs):

  admission   first come, first served; a request is admitted when a sequence slot is free and
              the cache can hold its whole prompt plus one generated token (+ the watermark
              when others run); the head of the queue blocks those behind it (:494-624, :659-697)
  portions    each running sequence that still has prompt left gets min(rest, budget) tokens;
              with `decode_first` one token of the budget is kept per decoding sequence
              (:340-400)
  decoding    every running sequence whose prompt is computed gets one row; if no page is left
              for it the newest running sequence is preempted (:401-455, :647-657)
  preemption  by recompute: all pages go back, the sequence returns to the FRONT of the queue
              and later prefills prompt and generated tokens again (:933-968)
  policy      `fcfs`, or `priority` (:206-219, :625-697): the waiting request with the smallest (priority,
              arrival) is served first, running sequences are served in that order too, a waiting request of
              better priority takes the slot or the pages of the worst running sequence (never of an equal one),
              and when a decode row finds no page the worst sequence gives way instead of the newest

  prefixes    with `prefix_cache` the cache manager keeps the full pages of what was computed, and a request that is
              admitted starts behind the longest prefix of its tokens that is known there (the reference's prefix cache,
              rust/engine/src/mem/prefix_cache.rs:414-520); a preempted sequence finds its own pages again this way
              unless the room was needed
  state       for a model whose layers keep state of fixed size per request (`state_checkpoints`): such state cannot be
              shared by pointing at pages, it has to be copied at the position where two requests part.  A prompt whose
              beginning may serve others (the prefix cache is on, or further answers to it wait) is cut so that one
              portion ends on its last page boundary; the engine copies the state there (`take_checkpoints`), and a
              request that starts behind shared pages gets the copy put into its slot before its first step
              (`take_restores`).  The reference does the same with its state checkpoints (scheduler.rs:383-388, :536-560,
              :598-612; rust/engine/src/runtime.rs:979-1011)
  multiples   `portion_multiple`: a portion that does not end its prompt ends on a multiple of so many tokens (mixers
              whose kernels work on fixed chunks of positions ask for it)

The scheduler does the cache bookkeeping (reserve at admission and before a decode row); the
step function commits what it ran.
"""
from __future__ import annotations

import math
from collections import deque
from dataclasses import dataclass, field
from typing import Deque, Dict, List, Optional, Tuple

from ..cache import CacheManager
from ..sampling.params import SamplingParams


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 16                  # scheduler.rs:225-248 defaults
    max_num_batched_tokens: int = 512
    decode_first: bool = False
    watermark_pages: int = 0
    max_partial_prefills: int = 0           # 0: no limit
    long_prefill_threshold: int = 0         # 0: no distinction
    max_long_partial_prefills: int = 1
    preemption: str = "recompute"
    policy: str = "fcfs"                    # fcfs | priority (smaller `SamplingParams.priority` first)
    prefix_cache: bool = False              # requests start behind the prefix of their tokens that the cache knows
    state_checkpoints: bool = False         # the model keeps state per request: shared beginnings need a copy of it
    portion_multiple: int = 1               # portions that do not end a prompt end on multiples of this

    def __post_init__(self):
        if self.max_num_seqs <= 0 or self.max_num_batched_tokens <= 0:
            raise ValueError("max_num_seqs and max_num_batched_tokens must be positive")
        if self.preemption not in ("recompute", "none"):
            raise ValueError("preemption must be 'recompute' or 'none'")
        if self.policy not in ("fcfs", "priority"):
            raise ValueError("scheduling policy must be 'fcfs' or 'priority'")
        if self.portion_multiple <= 0:
            raise ValueError("portion_multiple must be positive")


@dataclass
class Sequence:
    seq_id: int
    req_id: str
    tokens: List[int]                       # prompt, then generated tokens
    prompt_len: int
    sampling: SamplingParams
    num_computed: int = 0                   # tokens whose keys and values are in the cache
    prefill_target: int = 0                 # tokens to run as prompt (all tokens after a preemption)
    state: str = "waiting"                  # waiting | running | finished
    preempted: bool = False
    arrival: int = 0
    draws: int = 0                          # random draws taken so far
    seen: Optional[object] = None           # counts of the tokens so far, kept by the engine for requests with penalties
    choice: int = 0                         # which of the answers to its request's prompt this sequence is
    fork_from: Optional[int] = None         # a sequence that begins with the same tokens (the first answer, for the others)
    forks: bool = False                     # further answers will start behind this sequence's prompt
    checkpoint_at: Optional[int] = None     # tokens after which the model's per-request state is to be copied

    @property
    def output_len(self) -> int:
        return len(self.tokens) - self.prompt_len

    def remaining(self) -> int:
        return self.sampling.max_tokens - self.output_len


@dataclass
class ScheduledStep:
    prefill: List[Tuple[int, int, int]] = field(default_factory=list)    # (seq_id, start, count)
    decode: List[int] = field(default_factory=list)


class Scheduler:
    def __init__(self, cfg: SchedulerConfig, cache: CacheManager, max_model_len: int):
        self.cfg = cfg
        self.cache = cache
        self.max_model_len = max_model_len
        self.sequences: Dict[int, Sequence] = {}
        self.waiting: Deque[int] = deque()
        self.running: List[int] = []
        self.preemptions = 0
        self._arrivals = 0
        if cfg.prefix_cache:
            cache.enable_prefix_cache()
        # per-request state of the model (`state_checkpoints`): copies the engine took, by sequence: (tokens, copy);
        # what it has to copy after the step it is about to run, and what it has to put back before it
        self.state_copies: Dict[int, Tuple[int, object]] = {}
        self._checkpoints: List[Tuple[int, int]] = []
        self._restores: List[Tuple[int, object]] = []

    # ---- queue ----------------------------------------------------------------------------
    def add(self, seq: Sequence) -> None:
        seq.arrival = self._arrivals
        self._arrivals += 1
        seq.prefill_target = len(seq.tokens)
        seq.state = "waiting"
        self.sequences[seq.seq_id] = seq
        self.waiting.append(seq.seq_id)

    def has_work(self) -> bool:
        return bool(self.waiting or self.running)

    def _try_admit(self, sid: int) -> bool:
        seq = self.sequences[sid]
        if len(seq.tokens) > self.max_model_len:
            return False
        with_state = self.cfg.state_checkpoints
        self.cache.add_request(sid)
        total = len(seq.tokens) + 1
        watermark = self.cfg.watermark_pages if self.running else 0
        state = None
        if self.cfg.prefix_cache:
            # looked up without taking hold: a request that does not fit yet leaves the index as it was (its hits are
            # not counted, the pages it would use keep their place in the order in which unused ones are given up)
            known, idle = self.cache.probe_prefix(seq.tokens, with_state)
            missing = self.cache.pages_missing(sid, total)
            if any(m - known + watermark > self.cache.free_pages(g) - idle for g, m in enumerate(missing)):
                self.cache.free_request(sid)
                return False
            reused = self.cache.adopt_prefix(sid, seq.tokens, with_state)
            if with_state:
                reused, state = reused
        else:
            reused, state = self._share_with_source(seq)
            missing = self.cache.pages_missing(sid, total)
            if any(m + watermark > self.cache.free_pages(g) for g, m in enumerate(missing)):
                self.cache.free_request(sid)
                return False
        self.cache.reserve(sid, total)
        seq.num_computed = reused
        if state is not None:
            self._restores.append((sid, state))
        seq.checkpoint_at = None
        if with_state and (self.cfg.prefix_cache or seq.forks):
            unit = self._checkpoint_unit()
            boundary = (len(seq.tokens) - 1) // unit * unit          # the last token is always computed
            if unit > 0 and boundary > reused:
                seq.checkpoint_at = boundary
        return True

    def _checkpoint_unit(self) -> int:
        """State is copied where pages end and portions may end; 0: the page sizes of the groups differ."""
        sizes = {g.page_size for g in self.cache.groups}
        if len(sizes) > 1:
            return 0
        page, multiple = (sizes.pop() if sizes else 1), self.cfg.portion_multiple
        return page * multiple // math.gcd(page, multiple)

    def _share_with_source(self, seq: Sequence) -> Tuple[int, object]:
        """A further answer to a prompt starts behind the full pages of the first answer's sequence, as far as their
        tokens are the same, if that one still runs (the reference forks the block table and copies the last block,
        rust/engine/src/runtime.rs:437-460; here the last, partly filled page is computed again instead).  Where the
        model keeps state per request, only as far as the place where that state was copied.  Returns the tokens shared
        and the copy of the state to start from (None without)."""
        source = self.sequences.get(seq.fork_from) if seq.fork_from is not None else None
        if source is None or source.seq_id not in self.running:
            return 0, None
        limit = min(len(seq.tokens) - 1, len(source.tokens), source.num_computed)     # the last token is always computed
        state = None
        if self.cfg.state_checkpoints:
            tokens, state = self.state_copies.get(source.seq_id, (0, None))
            if state is None or tokens > limit:
                return 0, None
            limit = tokens
        same = limit if seq.tokens[:limit] == source.tokens[:limit] else 0
        while same < limit and seq.tokens[same] == source.tokens[same]:
            same += 1
        if state is not None and same != limit:
            return 0, None
        shared = self.cache.share_pages(source.seq_id, seq.seq_id, same)
        if state is not None and shared != limit:
            if shared:                                   # cannot be: the copy was taken where the source's pages end
                raise RuntimeError(f"{shared} tokens shared, the state was copied behind {limit}")
            return 0, None
        return shared, state

    def take_checkpoints(self) -> List[Tuple[int, int]]:
        """(sequence, tokens) of the sequences whose portion of the step just committed ended where their state is to be
        copied: the caller copies it now, before the next step, and hands it to `keep_checkpoint`."""
        due, self._checkpoints = self._checkpoints, []
        return due

    def keep_checkpoint(self, sid: int, tokens: int, state) -> None:
        seq = self.sequences.get(sid)
        if seq is None:
            return
        if seq.forks:
            self.state_copies[sid] = (tokens, state)
        if self.cfg.prefix_cache:
            self.cache.keep_state(sid, tokens, state)

    def take_restores(self) -> List[Tuple[int, object]]:
        """(sequence, copy of a state) for the sequences admitted since the last call that start behind a shared
        beginning: the caller puts the copy into the sequence's slot before it runs the step."""
        due, self._restores = self._restores, []
        return [(sid, state) for sid, state in due if sid in self.running]

    # ---- order ----------------------------------------------------------------------------
    def _key(self, sid: int) -> Tuple[int, int]:
        """The sequence with the smaller key goes first (scheduler.rs:625-631)."""
        seq = self.sequences[sid]
        return (seq.sampling.priority if self.cfg.policy == "priority" else 0, seq.arrival)

    def _ordered_running(self) -> List[int]:
        return sorted(self.running, key=self._key) if self.cfg.policy == "priority" else list(self.running)

    def _pick_waiting(self) -> Optional[int]:
        if not self.waiting:
            return None
        return min(self.waiting, key=self._key) if self.cfg.policy == "priority" else self.waiting[0]

    def _victim(self, needy: int) -> int:
        """Who gives way to `needy`: the last arrival under FCFS, the running sequence of the worst priority (the
        newest of them) otherwise (scheduler.rs:646-658)."""
        if self.cfg.policy == "priority":
            others = [sid for sid in self.running if sid != needy]
            return max(others, key=self._key) if others else needy
        return self.running[-1]

    def _admit_waiting(self) -> None:
        by_priority = self.cfg.policy == "priority" and self.cfg.preemption == "recompute"
        while True:
            sid = self._pick_waiting()
            if sid is None:
                break
            if len(self.running) >= self.cfg.max_num_seqs:
                # all slots taken: a waiting request of better priority takes the slot of the worst running sequence
                if not (by_priority and self.running and self._key(self._victim(sid))[0] > self._key(sid)[0]):
                    break
                self._preempt(self._victim(sid))
            ok = self.cache.free_slots() > 0 and self._try_admit(sid)
            if not ok and by_priority and self.running and self.cache.free_slots() > 0:
                victim = self._victim(sid)          # the pool is full: the pages of a running sequence of worse priority
                if self._key(victim)[0] > self._key(sid)[0]:
                    self._preempt(victim)
                    ok = self._try_admit(sid)
            if not ok:
                break                       # the request that is next in line blocks those behind it
            self.waiting.remove(sid)
            self.sequences[sid].state = "running"
            self.running.append(sid)

    def _remember(self, sid: int) -> None:
        """Tells the cache which tokens the sequence's full pages hold.  A negative id stands for a token that is not
        known yet (a step still runs); such tokens are at the end only."""
        if not self.cfg.prefix_cache:
            return
        tokens = self.sequences[sid].tokens
        known = len(tokens)
        while known > 0 and tokens[known - 1] < 0:
            known -= 1
        self.cache.remember_prefix(sid, tokens, known)

    def _preempt(self, sid: int) -> None:
        seq = self.sequences[sid]
        seq.preempted = True
        self.preemptions += 1
        self.cache.free_request(sid)
        seq.num_computed = 0
        seq.prefill_target = len(seq.tokens)
        seq.state = "waiting"
        seq.checkpoint_at = None
        self.state_copies.pop(sid, None)
        self.running.remove(sid)
        self.waiting.appendleft(sid)

    # ---- one step -------------------------------------------------------------------------
    def schedule(self) -> Optional[ScheduledStep]:
        self._admit_waiting()
        if not self.running:
            return None
        step = ScheduledStep()
        budget = self.cfg.max_num_batched_tokens
        decoders = sum(1 for sid in self.running
                       if self.sequences[sid].num_computed >= self.sequences[sid].prefill_target
                       and self.sequences[sid].remaining() > 0)
        prefill_budget = max(1, budget - decoders) if self.cfg.decode_first else budget
        long_prefills = 0
        for sid in self._ordered_running():
            if prefill_budget == 0 or budget == 0:
                break
            if self.cfg.max_partial_prefills > 0 and len(step.prefill) >= self.cfg.max_partial_prefills:
                break
            seq = self.sequences[sid]
            todo = seq.prefill_target - seq.num_computed
            if todo <= 0:
                continue
            is_long = self.cfg.long_prefill_threshold > 0 and seq.prefill_target > self.cfg.long_prefill_threshold
            if is_long and long_prefills >= max(1, self.cfg.max_long_partial_prefills):
                continue
            chunk = min(todo, prefill_budget)
            if seq.checkpoint_at is not None and seq.num_computed < seq.checkpoint_at < seq.num_computed + chunk:
                chunk = seq.checkpoint_at - seq.num_computed     # state can only be copied between two portions
            if self.cfg.portion_multiple > 1 and chunk < todo:
                chunk -= (seq.num_computed + chunk) % self.cfg.portion_multiple
                if chunk <= 0:
                    continue                                     # no room for a whole multiple in this step
            if not self.cache.can_reserve(sid, seq.num_computed + chunk):
                break
            self.cache.reserve(sid, seq.num_computed + chunk)
            step.prefill.append((sid, seq.num_computed, chunk))
            budget -= chunk
            prefill_budget -= chunk
            long_prefills += int(is_long)
        for sid in self._ordered_running():
            if sid not in self.running:
                continue                    # preempted by an earlier sequence of this loop
            seq = self.sequences[sid]
            if seq.num_computed < seq.prefill_target or seq.remaining() <= 0:
                continue
            if any(sid == p[0] for p in step.prefill):
                continue
            if budget == 0:
                break
            total = len(seq.tokens)         # the newest token has no keys yet: it is this row
            if not self.cache.can_reserve(sid, total):
                if self.cfg.preemption == "recompute" and len(self.running) > 1:
                    victim = self._victim(sid)
                    if victim != sid:
                        self._preempt(victim)
                        step.decode = [d for d in step.decode if d != victim]
                        step.prefill = [p for p in step.prefill if p[0] != victim]
                if not self.cache.can_reserve(sid, total):
                    continue
            self.cache.reserve(sid, total)
            budget -= 1
            step.decode.append(sid)
        if not step.prefill and not step.decode:
            return None
        return step

    # ---- after the step -------------------------------------------------------------------
    def commit_chunk(self, sid: int, count: int) -> None:
        seq = self.sequences[sid]
        seq.num_computed += count
        self._remember(sid)
        if seq.checkpoint_at is not None and seq.num_computed >= seq.checkpoint_at:
            if seq.num_computed == seq.checkpoint_at:
                self._checkpoints.append((sid, seq.checkpoint_at))
            seq.checkpoint_at = None

    def commit_decode(self, sid: int) -> None:
        seq = self.sequences[sid]
        seq.num_computed = len(seq.tokens) - 1      # the token just appended is the next decode row
        self._remember(sid)

    def finish(self, sid: int) -> None:
        if sid in self.running:
            self._remember(sid)
        seq = self.sequences.pop(sid)
        seq.state = "finished"
        self.state_copies.pop(sid, None)
        if sid in self.running:
            self.running.remove(sid)
        if sid in self.waiting:
            self.waiting.remove(sid)
        self.cache.free_request(sid)
