"""The engine: requests in, token events out.  `Engine` puts the scheduler and the sampler on
top of the step function, in the shape of the reference's runtime
(rust/engine/src/runtime.rs:365-467 `submit*`, :2141-2149 `step`, :2212-3150 `step_round`,
:3152-3168 `run_until_request_done`; driven without a server as in
rust/engine/examples/perf_decode.rs:24-46).
"""
from __future__ import annotations

import os
import time
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence as Seq, Tuple, Union

import torch

from ..config.files import read_config_json
from ..registry import model_spec_from_config
from ..sampling import SampleRequest, Sampler, SamplingParams
from ..weights.loader import load_checkpoint
from ..weights.random_init import random_tensors
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler, SchedulerConfig, Sequence


@dataclass
class TokenEvent:
    request_id: str
    token_id: int
    finished: bool
    finish_reason: Optional[str] = None     # "stop" | "length" | "timeout" (then no token comes with it: token_id -1)
    choice: int = 0                         # with `SamplingParams.n` > 1: which of the answers the token belongs to
    logprob: Optional[float] = None         # with `SamplingParams.logprobs`: of this token in the model's distribution
                                            # (with `logprobs_processed`: in the one it was drawn from)
    top_logprobs: Optional[List[Tuple[int, float]]] = None     # and the likeliest tokens, (id, log-probability)


@dataclass
class EngineStats:
    """Counters in the manner of the reference's BatchStats (runtime.rs:20-40)."""
    forward_calls: int = 0
    rows_total: int = 0
    max_rows: int = 0
    prefill_rows: int = 0
    decode_rows: int = 0
    preemptions: int = 0
    prefix_hit_tokens: int = 0     # prompt tokens that were not computed because the cache knew them
    scheduler_s: float = 0.0
    forward_s: float = 0.0
    postprocess_s: float = 0.0


PENDING = -1      # stands in a sequence's token list for a token that is still on the device


@dataclass
class _InFlight:
    """A launched step whose tokens have not been read: sequence ids in row order, where each
    token goes in its sequence, the device tensor that will hold them (the next step takes its input from there),
    and the copy of them to the host that was queued right behind the step."""
    sampled: List[int]
    at: List[int]
    tokens: torch.Tensor
    on_host: object = None
    logprobs: object = None      # what `Sampler.finish_logprobs` takes, when a row asked for log-probabilities


class Engine:
    def __init__(self, model: Union[str, None] = None, *, config: Optional[dict] = None, seed: int = 0,
                 dtype: str = "bfloat16", device: str = "cuda:0", ctx: Optional[int] = None, max_seqs: int = 16,
                 max_batched_tokens: int = 512, block_size: int = 16, num_blocks: Optional[int] = None,
                 gpu_memory_utilization: float = 0.90, decode_first: bool = True, kv_watermark_blocks: int = 0,
                 max_num_partial_prefills: int = 0, long_prefill_token_threshold: int = 0, max_long_partial_prefills: int = 1,
                 preemption_mode: str = "recompute", eos_token_ids: Optional[Seq[int]] = None,
                 random_weights_on_device: bool = False, ops=None, ahead: bool = True, check_layers: int = 0,
                 scheduling_policy: str = "fcfs", prefix_cache: Optional[bool] = None, decode_weight_tiles="auto"):
        """`model`: a folder with config.json and safetensors; or `config` (a config.json dict)
        with `seed` for random weights (drawn on the host, or on the device with a stream of its
        own when `random_weights_on_device`: large models).  Option names follow the reference's server flags
        (rust/engine/src/bin/serve.rs:530-557, :681-782): ctx, max_seqs, max_batched_tokens,
        gpu_memory_utilization, kv_watermark_blocks, max_num_partial_prefills,
        long_prefill_token_threshold, max_long_partial_prefills, preemption_mode, scheduling_policy (`fcfs`, or `priority`: requests with the
        smaller `SamplingParams.priority` first, and a waiting one of better priority takes the place of the worst
        running one).  `prefix_cache` (the reference's environment switch FLLM_PREFIX_CACHE, rust/engine/src/runtime.rs:193-206,
        is read when it is None; off by default here): full cache pages outlive their request, and a request that begins
        with the same tokens starts behind them.  Its tokens are then the same as without only up to rounding, as
        with any other change of how tokens are batched.

        `ahead` (the default; False: every `step()` waits for its own tokens and returns them, and the host's work per
        step adds to the step): a step is launched before the tokens of the step before it have reached the host
        (the reference's ahead step, rust/engine/src/rust_decoder.rs:1165-1266): the device takes
        them from the earlier step's output, the host plans the next step while the device runs
        this one, and `step()` returns the events of the step before.  A request that stops at a
        token (end of sequence, stop id) has one more row in flight by then; that row is dropped.

        `decode_weight_tiles` (True, False, "auto": within half of the memory that is free once the weights are placed):
        second copies of the layers' matrices in the order decode steps read them (`Runtime.tile_for_decode`).

        `check_layers`: the first so many steps run every layer also with the plain kernels and print, layer by
        layer, how far the two are apart, the largest value, a checksum and NaN/Inf counts (`runner.check_layers`)."""
        if (model is None) == (config is None):
            raise ValueError("give either a model folder or a config for random weights")
        if model is not None:
            config = read_config_json(model)
        typed, spec = model_spec_from_config(config)
        if model is not None:
            tensors = load_checkpoint(model, spec)
        else:
            from .runner import parse_dtype
            tensors = random_tensors(spec, seed, parse_dtype(dtype), device=device if random_weights_on_device else "cpu")
        self.runner = ModelRunner(spec, tensors, dtype=dtype, device=device, page_size=block_size, num_pages=num_blocks,
                                  max_requests=max_seqs, max_context=ctx, memory_utilization=gpu_memory_utilization,
                                  ops=ops, typed_config=typed, max_step_tokens=max_batched_tokens,
                                  decode_weight_tiles=decode_weight_tiles, consume_tensors=True)
        del tensors
        self.config = typed
        self.max_model_len = self.runner.max_context
        if prefix_cache is None:
            prefix_cache = os.environ.get("FLLM_PREFIX_CACHE", "").strip().lower() in ("1", "on", "true", "yes")
        self.scheduler = Scheduler(
            SchedulerConfig(max_num_seqs=max_seqs, max_num_batched_tokens=max_batched_tokens, decode_first=decode_first,
                            watermark_pages=kv_watermark_blocks, max_partial_prefills=max_num_partial_prefills,
                            long_prefill_threshold=long_prefill_token_threshold,
                            max_long_partial_prefills=max_long_partial_prefills, preemption=preemption_mode,
                            policy=scheduling_policy, prefix_cache=bool(prefix_cache),
                            state_checkpoints=self.runner.model.has_state,
                            portion_multiple=self.runner.model.portion_multiple),
            self.runner.cache, self.max_model_len)
        self.sampler = Sampler(self.runner.rt)
        if eos_token_ids is None:
            eos_token_ids = getattr(typed, "eos_token_ids", ()) or ()
            if not eos_token_ids and model is not None and os.path.isdir(model):
                from ..config.files import generation_eos_ids
                eos_token_ids = generation_eos_ids(model)
        self.eos_token_ids = tuple(int(t) for t in eos_token_ids)
        self.stats = EngineStats()
        self._requests: Dict[str, List[int]] = {}        # the sequences of a request that have not ended: one an answer
        self._followers: Dict[int, List[Sequence]] = {}  # further answers that wait until the first one's prompt is computed
        self._deadlines: Dict[str, float] = {}
        self._next_seq = 0
        self.ahead = bool(ahead)
        self._in_flight: Optional[_InFlight] = None
        self.layer_check = self.runner.check_layers(check_layers) if check_layers > 0 else None

    # ---- requests -------------------------------------------------------------------------
    def add_request(self, request_id: str, prompt_token_ids: Seq[int], sampling: Optional[SamplingParams] = None) -> int:
        sampling = sampling or SamplingParams()
        prompt = [int(t) for t in prompt_token_ids]
        if not request_id or not prompt:
            raise ValueError("request id, prompt tokens, and max_tokens must be non-empty")
        if len(prompt) + sampling.max_tokens > self.max_model_len:
            raise ValueError("prompt plus max_tokens exceeds the configured model context")
        if request_id in self._requests:
            raise ValueError(f"request id already active: {request_id}")
        for t in prompt:
            if not 0 <= t < self.runner.vocab_size:
                raise ValueError(f"token id {t} is outside [0, {self.runner.vocab_size})")
        sid = self._next_seq
        self._next_seq += sampling.n
        self.scheduler.add(Sequence(seq_id=sid, req_id=request_id, tokens=prompt, prompt_len=len(prompt), sampling=sampling,
                                    forks=sampling.n > 1))
        self._requests[request_id] = list(range(sid, sid + sampling.n))
        if sampling.n > 1:
            # the other answers join when the first one's prompt is in the cache, and start behind its full pages
            # (where layers keep state of their own per request: behind the place where that state was copied)
            self._followers[sid] = [Sequence(seq_id=sid + k, req_id=request_id, tokens=list(prompt), prompt_len=len(prompt),
                                             sampling=sampling.for_choice(k), choice=k, fork_from=sid)
                                    for k in range(1, sampling.n)]
        self._deadlines.pop(request_id, None)
        if sampling.timeout_secs is not None:
            self._deadlines[request_id] = time.monotonic() + float(sampling.timeout_secs)
        return sid

    def expire_requests(self) -> List[str]:
        """Gives up the requests whose `timeout_secs` have passed since they were added, waiting included, and returns
        their ids; what they hold goes back (rust/engine/src/runtime.rs:1222-1232).  `step` calls it."""
        if not self._deadlines:
            return []
        now = time.monotonic()
        self._deadlines = {rid: d for rid, d in self._deadlines.items() if rid in self._requests}     # the others have ended
        expired = sorted(rid for rid, deadline in self._deadlines.items() if deadline <= now)
        for rid in expired:
            del self._deadlines[rid]
            self.abort_request(rid)
        return expired

    def abort_request(self, request_id: str) -> None:
        for sid in self._requests.pop(request_id, ()):
            self._followers.pop(sid, None)
            if sid in self.scheduler.sequences:
                self.scheduler.finish(sid)

    def clear_prefix_cache(self) -> int:
        """Gives up the cached prefixes that no request uses (rust/engine/src/runtime.rs:1175-1180); returns the pages freed."""
        return self.runner.cache.clear_prefixes()

    def has_unfinished(self) -> bool:
        return self.scheduler.has_work() or self._in_flight is not None

    # ---- one round ------------------------------------------------------------------------
    def step(self) -> List[TokenEvent]:
        """Schedules and runs one step.  Returns the tokens it produced; with `ahead`, those of the
        step before, while this one runs."""
        timed_out = [TokenEvent(rid, -1, True, "timeout") for rid in self.expire_requests()]
        if timed_out:
            return timed_out + self._step()
        return self._step()

    def _step(self) -> List[TokenEvent]:
        t0 = time.perf_counter()
        plan = self.scheduler.schedule()
        t1 = time.perf_counter()
        self.stats.scheduler_s += t1 - t0
        self.stats.preemptions = self.scheduler.preemptions
        self.stats.prefix_hit_tokens = self.runner.cache.prefix_hit_tokens
        earlier, self._in_flight = self._in_flight, None
        if plan is None:
            if earlier is not None:
                return self._resolve(earlier)
            if self.scheduler.has_work():
                raise RuntimeError("scheduler could not make progress with the available KV pool")
            return []
        seqs = self.scheduler.sequences
        entries: List[StepEntry] = []
        sampled: List[int] = []                  # sequence ids whose row gives a token, in row order
        row_of = {sid: r for r, sid in enumerate(earlier.sampled)} if earlier is not None else {}
        for sid, start, count in plan.prefill:
            seq = seqs[sid]
            last = start + count == seq.prefill_target
            entries.append(StepEntry(sid, seq.tokens[start:start + count], [count - 1] if last else []))
            if last:
                sampled.append(sid)
        for sid in plan.decode:
            token = seqs[sid].tokens[-1]
            entries.append(StepEntry(sid, [token], [0], carry=row_of[sid] if token == PENDING else None))
            sampled.append(sid)
        for sid, state in self.scheduler.take_restores():         # requests that start behind a shared beginning
            self.runner.restore_state(sid, state)
        try:
            logits = self.runner.step(entries, previous_tokens=earlier.tokens if earlier is not None else None)
        except Exception:
            # nothing was launched: the earlier step stays in flight, so that its tokens still replace their
            # placeholders (the next call schedules again)
            self._in_flight = earlier
            raise
        self.stats.prefill_rows += sum(count for _, _, count in plan.prefill)
        self.stats.decode_rows += len(plan.decode)
        rows = sum(len(e.tokens) for e in entries)
        self.stats.forward_calls += 1
        self.stats.rows_total += rows
        self.stats.max_rows = max(self.stats.max_rows, rows)
        requests = [SampleRequest(seqs[sid].sampling, seqs[sid].sampling.seed_for(sid), seqs[sid].draws) for sid in sampled]
        wants_logprobs = [r for r, sid in enumerate(sampled) if seqs[sid].sampling.logprobs is not None]
        wants_processed = [r for r in wants_logprobs if seqs[sampled[r]].sampling.logprobs_processed]
        wants_raw = [r for r in wants_logprobs if r not in wants_processed]
        adjusting = any(seqs[sid].sampling.adjusts_logits(seqs[sid].output_len) for sid in sampled)
        as_given = logits.clone() if wants_raw and adjusting else logits
        if adjusting:
            self._adjust(logits, sampled, row_of, earlier)
        launched = _InFlight(sampled, [], self.sampler.launch(logits, requests))
        # queued now, before the next step is launched behind it: reading these tokens must not wait for that step
        launched.on_host = self.sampler.start_read(launched.tokens)
        if wants_logprobs:
            top = max(seqs[sampled[r]].sampling.logprobs for r in wants_logprobs)
            launched.logprobs = self.sampler.start_logprobs(as_given, launched.tokens, wants_raw, top, processed=wants_processed,
                                                            seen=logits, requests=requests)
        # What does not depend on the tokens' values: the sequences grow by one (a placeholder until the
        # token is read), the prompt portions count as computed.
        for sid, _, count in plan.prefill:
            self.scheduler.commit_chunk(sid, count)
        for sid, tokens in self.scheduler.take_checkpoints():     # copied now, on the step's stream, before the next step
            self.scheduler.keep_checkpoint(sid, tokens, self.runner.snapshot_state(sid))
        for sid in sampled:
            seq = seqs[sid]
            launched.at.append(len(seq.tokens))
            seq.tokens.append(PENDING)
            if not seq.sampling.greedy:
                seq.draws += 1
            self.scheduler.commit_decode(sid)
            for follower in self._followers.pop(sid, ()):       # the prompt is computed: the other answers may begin
                self.scheduler.add(follower)
        if self.ahead:
            self._in_flight = launched
            events = self._resolve(earlier) if earlier is not None else []
        else:
            events = self._resolve(launched)
        self.stats.forward_s += time.perf_counter() - t1
        return events

    def _adjust(self, logits, sampled: List[int], row_of: Dict[int, int], earlier: Optional[_InFlight]) -> None:
        """Penalties, biases and blocked ids of the requests that ask for any, on the step's logits before a token is
        chosen.  A request whose newest token is still a placeholder (the step in flight chose it) has it counted on
        the device, from that step's tokens."""
        seqs = self.scheduler.sequences
        from ..sampling.adjust import SeenTokens, row_for
        rows = []
        for sid in sampled:
            seq = seqs[sid]
            pending = row_of[sid] if seq.tokens[-1] == PENDING else None
            if seq.seen is None and seq.sampling.penalizes:
                seq.seen = SeenTokens()
            rows.append(row_for(seq.sampling, seq.tokens, seq.prompt_len, pending, self.eos_token_ids, seq.seen))
        self.sampler.adjust(logits, rows, earlier.tokens if earlier is not None else None)

    def _resolve(self, step: _InFlight) -> List[TokenEvent]:
        """Reads a launched step's tokens (waits for the device), puts them where the placeholders
        are and finishes the requests that end with them."""
        t0 = time.perf_counter()
        tokens = self.sampler.finish_read(step.on_host)
        logprobs = self.sampler.finish_logprobs(step.logprobs) if step.logprobs is not None else {}
        seqs = self.scheduler.sequences
        events: List[TokenEvent] = []
        for row, (sid, at, token) in enumerate(zip(step.sampled, step.at, tokens)):
            seq = seqs.get(sid)
            if seq is None:
                continue                         # finished or aborted while this row was in flight
            seq.tokens[at] = token
            hit_stop = seq.sampling.stops_on(token, self.eos_token_ids)
            hit_limit = at + 1 - seq.prompt_len >= seq.sampling.max_tokens
            reason = "stop" if hit_stop else ("length" if hit_limit else None)
            if reason:
                self.scheduler.finish(sid)
                left = self._requests.get(seq.req_id)
                if left is not None:
                    left.remove(sid)
                    if not left:
                        del self._requests[seq.req_id]
            event = TokenEvent(seq.req_id, token, reason is not None, reason, choice=seq.choice)
            if row in logprobs:
                event.logprob, alternatives = logprobs[row]
                event.top_logprobs = alternatives[:seq.sampling.logprobs]
            events.append(event)
        self.stats.postprocess_s += time.perf_counter() - t0
        return events

    # ---- before the first request ----------------------------------------------------------
    def warm_up(self, context_bounds: Optional[Seq[int]] = None) -> int:
        """Runs a few synthetic requests so that what is built at first use exists before the first real request
        (rust/engine/src/runtime.rs:1085-1173): the decode graph of every batch size that `max_seqs` sequences can
        reach, the sampler, prompt portions of 128 to 2,048 tokens; then captures the same graphs for longer
        contexts (`context_bounds`, by default the powers of two up to the context or 32,768).  Nothing of it
        stays: every request is finished, the counters are put back.  Returns the number of requests run."""
        if self.scheduler.has_work() or self._in_flight is not None:
            return 0
        from .runner import GRAPH_BUCKETS
        saved = EngineStats(**vars(self.stats))
        max_seqs = self.scheduler.cfg.max_num_seqs
        budget = self.scheduler.cfg.max_num_batched_tokens
        room = self.max_model_len
        vocab = self.runner.vocab_size
        sizes = [b for b in GRAPH_BUCKETS if b <= max_seqs]
        if max_seqs not in sizes:
            sizes.append(max_seqs)
        plan = [(rows, 8, 4, False) for rows in sizes] + [(1, 8, 4, True), (min(max_seqs, 16), 8, 4, True)]
        plan += [(1, tokens, 1, False) for tokens in (128, 256, 512, 1024, 2048) if tokens + 8 <= room and tokens <= budget]
        ran = serial = 0
        for count, prompt_len, new_tokens, sampled in plan:
            if prompt_len + new_tokens > room:
                continue
            names = []
            for _ in range(count):
                serial += 1
                prompt = [(serial * 131 + j * 17) % vocab for j in range(prompt_len)]
                params = SamplingParams(max_tokens=new_tokens, temperature=0.7 if sampled else 0.0,
                                        top_p=0.9 if sampled else 1.0, ignore_eos=True, seed=serial)
                name = f"__warmup_{serial}"
                self.add_request(name, prompt, params)
                names.append(name)
            try:
                while any(n in self._requests for n in names):
                    self.step()
                while self._in_flight is not None:
                    self.step()
            except Exception:
                for n in names:
                    self.abort_request(n)
                self._in_flight = None
                self.stats = saved
                raise
            ran += len(names)
        if context_bounds is None:
            context_bounds = []
            bound = 512
            while bound <= min(room, 32768):
                context_bounds.append(bound)
                bound *= 2
        self.runner.capture_graphs(sizes, context_bounds)
        self.stats = saved
        self.scheduler.preemptions = saved.preemptions
        self.runner.cache.clear_prefixes()
        self.runner.cache.prefix_hit_tokens = saved.prefix_hit_tokens
        return ran

    # ---- whole requests -------------------------------------------------------------------
    def generate(self, prompts: Seq[Seq[int]], sampling: Union[SamplingParams, Seq[SamplingParams], None] = None
                 ) -> List[List[int]]:
        """Generated token ids of every prompt (token ids in, token ids out); for a prompt whose parameters ask for
        n > 1 answers, the list of its n answers."""
        if sampling is None or isinstance(sampling, SamplingParams):
            sampling = [sampling or SamplingParams()] * len(prompts)
        if len(sampling) != len(prompts):
            raise ValueError("one SamplingParams per prompt is required")
        names = []
        for i, (p, s) in enumerate(zip(prompts, sampling)):
            name = f"generate-{self._next_seq}-{i}"
            self.add_request(name, p, s)
            names.append(name)
        outputs: Dict[str, List[List[int]]] = {n: [[] for _ in range(s.n)] for n, s in zip(names, sampling)}
        while any(n in self._requests for n in names):
            for ev in self.step():
                if ev.request_id in outputs and ev.token_id >= 0:
                    outputs[ev.request_id][ev.choice].append(ev.token_id)
        return [outputs[n][0] if s.n == 1 else outputs[n] for n, s in zip(names, sampling)]
