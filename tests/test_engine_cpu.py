"""The step function, the scheduler and generation on the CPU, with the plain kernels of
tests/reference_ops.py in place of the HIP library: what is tested here is the engine's own
logic (batches, pages, portions, preemption), not the kernels."""
import math

import numpy as np
import pytest
import torch

import plain_llama
import tiny_configs as tc
import trace_tools as tt
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams
from fllm_amd.cache import OutOfPages
from fllm_amd.engine import ModelRunner, StepEntry, StepError
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights import random_tensors


def runner_for(name, max_tokens, **kw):
    cfg = tc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    tensors = random_tensors(spec, 7, torch.float32, with_optional=(name == "C"))
    r = ModelRunner(spec, tensors, dtype="float32", device="cpu", page_size=tc.PAGE_SIZES[name], max_tokens=max_tokens,
                    max_requests=8, ops=ReferenceOps(), **kw)
    return cfg, tc.to_float64(tensors), r


@pytest.mark.parametrize("name,lengths", [("A", [5, 17, 40]), ("C", [30, 70]), ("F", [20, 70]), ("G", [49, 60])])
@pytest.mark.parametrize("family", ["whole", "last32", "portions", "mixed"])
def test_every_way_of_cutting_gives_the_plain_logits(tmp_path, name, lengths, family):
    requests = {f"r{i}": tc.random_ids(n, tc.CONFIGS[name]["vocab_size"], 50 + i) for i, n in enumerate(lengths)}
    steps = {"whole": tt.whole, "last32": lambda r: tt.last_tokens_one_by_one(r, 8), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=2, decode_tail=5, refeed=[f"r{len(lengths) - 1}"])}[family](requests)
    steps = tt.number(steps)
    cfg, w64, runner = runner_for(name, tt.live_tokens_bound(steps, round_to=16))
    given_up = {}
    got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path), given_up)
    assert (len(given_up) == 1) == (family == "mixed")
    for rid, feedings in given_up.items():          # ended half way and fed again from the first token: the same logits
        assert np.array_equal(feedings[0], got[rid][:len(feedings[0])])
    for rid, toks in requests.items():
        want = plain_llama.forward(cfg, w64, toks)
        assert np.abs(got[rid] - want).max() <= 2e-5 * np.abs(want).max(), (family, rid)
    runner.cache.check_invariants()
    assert all(p.available == p.num_pages for p in runner.cache.pools)


def test_step_refuses_bad_batches():
    cfg, _, r = runner_for("A", 64)
    with pytest.raises(StepError, match="at least one entry"):
        r.step([])
    with pytest.raises(StepError, match="no tokens"):
        r.step([StepEntry("a", [], [])])
    with pytest.raises(StepError, match="outside"):
        r.step([StepEntry("a", [256], [0])])
    with pytest.raises(StepError, match="wants logits"):
        r.step([StepEntry("a", [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        r.step([StepEntry("a", [1], [0]), StepEntry("a", [2], [0])])
    with pytest.raises(StepError, match="context"):
        r.step([StepEntry("a", [1] * 129, [])])
    assert not r.cache.has_request("a")
    with pytest.raises(OutOfPages):
        r.step([StepEntry("a", [1] * 40, []), StepEntry("b", [1] * 40, [])])     # 64 tokens of cache
    assert not r.cache.has_request("a") and not r.cache.has_request("b")          # nothing changed
    r.cache.check_invariants()
    out = r.step([StepEntry("a", [1, 2, 3], [])])
    assert out.shape == (0, 256) and r.length("a") == 3


def make_engine(name="A", **kw):
    opts = dict(dtype="float32", device="cpu", ctx=tc.CONFIGS[name]["max_position_embeddings"], max_seqs=4,
                max_batched_tokens=16, block_size=tc.PAGE_SIZES[name], num_blocks=64, ops=ReferenceOps())
    opts.update(kw)
    return Engine(config=tc.CONFIGS[name], seed=1, **opts)


def plain_greedy(name, prompt, count):
    cfg = tc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    seq = list(prompt)
    for _ in range(count):
        seq.append(plain_llama.greedy(plain_llama.forward(cfg, w64, seq)[-1]))
    return seq[len(prompt):]


PROMPTS_A = [tc.random_ids(n, 256, 10 + n) for n in (5, 17, 31)]


def test_greedy_generation_matches_the_plain_implementation():
    """The workload of the first tiny configuration: prompts of 5/17/31 tokens, 16 greedy tokens each."""
    outs = make_engine().generate(PROMPTS_A, SamplingParams(max_tokens=16))
    assert outs == [plain_greedy("A", p, 16) for p in PROMPTS_A]


def test_few_pages_preempt_and_give_the_same_tokens():
    roomy = make_engine().generate(PROMPTS_A, SamplingParams(max_tokens=16))
    tight = make_engine(num_blocks=5)
    assert tight.generate(PROMPTS_A, SamplingParams(max_tokens=16)) == roomy
    assert tight.stats.preemptions >= 1
    tight.runner.cache.check_invariants()


def test_no_progress_is_an_error():
    engine = make_engine(num_blocks=2, max_seqs=1)          # 32 tokens of cache
    engine.add_request("a", tc.random_ids(30, 256, 1), SamplingParams(max_tokens=8))
    with pytest.raises(RuntimeError, match="could not make progress"):
        for _ in range(20):
            engine.step()


def test_seeded_sampling_is_reproducible_and_ignores_the_neighbours():
    """The second tiny configuration's workload in small: chunked prefill mixed with decode,
    temperature 0.8 from a fixed seed."""
    params = SamplingParams(max_tokens=6, temperature=0.8, top_p=0.95, seed=1234)
    prompts = [tc.random_ids(n, 512, 20 + n) for n in (1, 9, 40)]
    alone = [make_engine("B", max_batched_tokens=32).generate([p], params)[0] for p in prompts]
    together = make_engine("B", max_batched_tokens=32).generate(prompts, params)
    assert together == alone
    assert make_engine("B", max_batched_tokens=32).generate(prompts, params) == together
    other = make_engine("B", max_batched_tokens=32).generate(prompts, SamplingParams(max_tokens=6, temperature=0.8, seed=99))
    assert other != together


def test_finish_reasons_and_request_checks():
    engine = make_engine()
    first = plain_greedy("A", PROMPTS_A[0], 3)
    engine.add_request("stop", PROMPTS_A[0], SamplingParams(max_tokens=16, stop_token_ids=(first[2],)))
    engine.add_request("length", PROMPTS_A[0], SamplingParams(max_tokens=2))
    events = []
    while engine.has_unfinished():
        events += engine.step()
    done = {e.request_id: e for e in events if e.finished}
    assert done["stop"].finish_reason == "stop" and done["stop"].token_id == first[2]
    assert done["length"].finish_reason == "length"
    assert [e.token_id for e in events if e.request_id == "stop"] == first
    with pytest.raises(ValueError, match="non-empty"):
        engine.add_request("x", [], SamplingParams())
    with pytest.raises(ValueError, match="exceeds the configured model context"):
        engine.add_request("x", [1] * 120, SamplingParams(max_tokens=16))
    engine.add_request("dup", [1, 2], SamplingParams(max_tokens=4))
    with pytest.raises(ValueError, match="already active"):
        engine.add_request("dup", [1, 2], SamplingParams(max_tokens=4))
    engine.abort_request("dup")
    assert not engine.has_unfinished()
    engine.runner.cache.check_invariants()


def test_eos_from_config_stops_unless_ignored():
    cfg = dict(tc.TINY_A)
    first = plain_greedy("A", PROMPTS_A[1], 2)
    cfg["eos_token_id"] = first[1]
    base = dict(dtype="float32", device="cpu", ctx=128, max_seqs=2, max_batched_tokens=32, block_size=16, num_blocks=16,
                ops=ReferenceOps())
    assert Engine(config=cfg, seed=1, **base).generate([PROMPTS_A[1]], SamplingParams(max_tokens=8)) == [first]
    ignored = Engine(config=cfg, seed=1, **base).generate([PROMPTS_A[1]], SamplingParams(max_tokens=8, ignore_eos=True))
    assert len(ignored[0]) == 8 and ignored[0][:2] == first


# ---- steps launched ahead of the tokens of the step before ----------------------------------
def test_ahead_generation_gives_the_same_tokens():
    """Greedy and seeded sampling, prompt portions mixed with decode rows, few pages with preemption:
    launching a step before the last one's tokens are read changes no token."""
    greedy = SamplingParams(max_tokens=16)
    assert make_engine(ahead=True).generate(PROMPTS_A, greedy) == [plain_greedy("A", p, 16) for p in PROMPTS_A]
    tight = make_engine(num_blocks=5, ahead=True)
    assert tight.generate(PROMPTS_A, greedy) == make_engine().generate(PROMPTS_A, greedy)
    assert tight.stats.preemptions >= 1
    tight.runner.cache.check_invariants()
    params = SamplingParams(max_tokens=6, temperature=0.8, top_p=0.95, seed=1234)
    prompts = [tc.random_ids(n, 512, 20 + n) for n in (1, 9, 40)]
    assert (make_engine("B", max_batched_tokens=32, ahead=True).generate(prompts, params)
            == make_engine("B", max_batched_tokens=32).generate(prompts, params))


def test_ahead_events_come_one_step_later_and_stop_where_they_should():
    first = plain_greedy("A", PROMPTS_A[0], 5)
    engine = make_engine(ahead=True)
    engine.add_request("stop", PROMPTS_A[0], SamplingParams(max_tokens=16, stop_token_ids=(first[2],)))
    engine.add_request("length", PROMPTS_A[1], SamplingParams(max_tokens=2))
    engine.add_request("long", PROMPTS_A[0], SamplingParams(max_tokens=5))
    assert engine.step() == []                       # the first step is in flight: nothing to hand out yet
    events = []
    while engine.has_unfinished():
        events += engine.step()
    by_request = {}
    for e in events:
        by_request.setdefault(e.request_id, []).append(e)
    assert [e.token_id for e in by_request["stop"]] == first[:3]          # the row launched past the stop token is dropped
    assert by_request["stop"][-1].finish_reason == "stop"
    assert len(by_request["length"]) == 2 and by_request["length"][-1].finish_reason == "length"
    assert [e.token_id for e in by_request["long"]] == first and by_request["long"][-1].finish_reason == "length"
    assert all(not e.finished for evs in by_request.values() for e in evs[:-1])
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == []


def test_ahead_asks_for_a_steps_tokens_before_the_next_step_is_launched():
    """The copy of a step's tokens to the host is queued right behind that step, before the next one is launched: on
    the device's one stream a copy queued later would wait for the next step, and nothing would run ahead."""
    engine = make_engine(ahead=True)
    order = []
    run_step, start_read, finish_read = engine.runner.step, engine.sampler.start_read, engine.sampler.finish_read

    def spy_step(*a, **k):
        order.append("launch")
        return run_step(*a, **k)

    def spy_start(tokens):
        order.append("ask")
        return start_read(tokens)

    def spy_finish(pending):
        order.append("read")
        return finish_read(pending)

    engine.runner.step, engine.sampler.start_read, engine.sampler.finish_read = spy_step, spy_start, spy_finish
    engine.add_request("a", PROMPTS_A[0], SamplingParams(max_tokens=3))
    while engine.has_unfinished():
        engine.step()
    assert order[:5] == ["launch", "ask", "launch", "ask", "read"]
    assert order.count("ask") == order.count("read") == order.count("launch")
    for i, what in enumerate(order):              # every read follows the launch AND the asking of a later step, or ends the run
        if what == "read":
            assert order[:i].count("ask") >= order[:i + 1].count("read")


def test_ahead_abort_drops_the_row_in_flight():
    engine = make_engine(ahead=True)
    engine.add_request("a", PROMPTS_A[0], SamplingParams(max_tokens=8))
    engine.add_request("b", PROMPTS_A[1], SamplingParams(max_tokens=8))
    engine.step()
    engine.step()
    engine.abort_request("a")
    events = []
    while engine.has_unfinished():
        events += engine.step()
    assert all(e.request_id == "b" for e in events)
    assert [e.token_id for e in events][-3:] == plain_greedy("A", PROMPTS_A[1], 8)[-3:]
    engine.runner.cache.check_invariants()


def test_ahead_step_that_fails_keeps_the_step_before_in_flight():
    """A step that raises launched nothing: the tokens of the step before still replace their placeholders,
    and generation goes on as if the failed call had not happened."""
    want = plain_greedy("A", PROMPTS_A[0], 6)
    engine = make_engine(ahead=True)
    engine.add_request("a", PROMPTS_A[0], SamplingParams(max_tokens=6))
    engine.step()
    engine.step()
    real_step, calls = engine.runner.step, []

    def failing_once(entries, previous_tokens=None):
        if not calls:
            calls.append(1)
            raise OutOfPages("forced by the test")
        return real_step(entries, previous_tokens=previous_tokens)

    engine.runner.step = failing_once
    with pytest.raises(OutOfPages):
        engine.step()
    events = []
    while engine.has_unfinished():
        events += engine.step()
    seq_tokens = [e.token_id for e in events]
    assert seq_tokens == want[-len(seq_tokens):] and len(seq_tokens) >= 4
    assert events[-1].finished
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == []


def test_warm_up_leaves_nothing_behind():
    """Synthetic requests of every batch size run before the first real one; afterwards no request, no page and no
    count of theirs is left, and generation gives what it gives without a warm-up."""
    engine = make_engine(max_seqs=4, num_blocks=64)
    ran = engine.warm_up()
    assert ran >= 1 + 2 + 4 + 1 + 4                      # batch sizes 1, 2, 4, and the sampled runs
    assert engine.stats.forward_calls == 0 and engine.stats.rows_total == 0
    assert not engine.has_unfinished() and engine.runner.cache.requests() == []
    assert all(p.available == p.num_pages for p in engine.runner.cache.pools)
    engine.runner.cache.check_invariants()
    greedy = SamplingParams(max_tokens=8)
    assert engine.generate(PROMPTS_A, greedy) == make_engine(max_seqs=4, num_blocks=64).generate(PROMPTS_A, greedy)
    busy = make_engine()
    busy.add_request("x", PROMPTS_A[0], greedy)
    assert busy.warm_up() == 0                            # only before the first request


def test_layer_check_counts_bad_values_per_layer():
    import io
    log = io.StringIO()
    engine = make_engine(check_layers=1)
    engine.layer_check.out = log
    engine.generate([PROMPTS_A[0]], SamplingParams(max_tokens=3))
    reports = engine.layer_check.reports
    assert [r.entry for r in reports] == [0, 1] and all(r.step == 0 and r.rows == len(PROMPTS_A[0]) for r in reports)
    assert all(r.bad_values == 0 and r.distance is None and r.largest > 0 for r in reports)      # one kind of kernel here
    assert not engine.layer_check.active and log.getvalue().count("[layer-check] step 0") == 2
    assert "none beyond" in log.getvalue()
    # a weight that is not a number: the first layer that touches it is named
    broken = make_engine(check_layers=1)
    broken.layer_check.out = log
    broken.runner.model.blocks[1].feed_forward.w_down[3, 5] = float("nan")
    broken.generate([PROMPTS_A[0]], SamplingParams(max_tokens=1))
    assert [r.bad_values > 0 for r in broken.layer_check.reports] == [False, True]
    assert "first suspect: step 0, run entry 1" in log.getvalue()


def test_own_gate_up_beside_the_library_only_where_it_was_measured_faster():
    """Up to 32 rows and from 128 MiB of gate and up weights on, a step whose products go to the GEMM library keeps
    the own gate/up product with the SwiGLU epilogue; not below 17 rows (those steps take the fused kernels
    anyway), not for small matrices, not without the library."""
    from types import SimpleNamespace
    from fllm_amd.kernels import Ops
    big = torch.empty(0, dtype=torch.bfloat16).new_empty((2 * 14336, 4096), device="meta")
    small = torch.empty(0, dtype=torch.bfloat16).new_empty((2 * 8192, 2048), device="meta")
    ops = SimpleNamespace(library_gemm_from=17, OWN_GATE_UP_ROWS=Ops.OWN_GATE_UP_ROWS, OWN_GATE_UP_BYTES=Ops.OWN_GATE_UP_BYTES)
    prefers = lambda rows, w, o=ops: Ops.prefers_own_gate_up(o, rows, w)
    assert [prefers(r, big) for r in (16, 17, 32, 33, 64)] == [False, True, True, False, False]
    assert not prefers(24, small)
    assert not prefers(24, big, SimpleNamespace(library_gemm_from=None, OWN_GATE_UP_ROWS=32, OWN_GATE_UP_BYTES=1))


def test_rows_that_draw_from_all_tokens_are_told_as_the_kernel_tells_them():
    """What the sampler says it knows of its rows is judged on the float32 values of the row records: a temperature a
    hair above the greedy limit, or a top-p a hair below one, rounds across the limit there."""
    from fllm_amd.sampling.sampler import draws_from_all
    P = SamplingParams
    assert draws_from_all(P(temperature=0.8), 100) and draws_from_all(P(temperature=0.8, top_k=100), 100)
    assert draws_from_all(P(temperature=0.8, top_p=1.0), 100)
    assert not draws_from_all(P(temperature=0.0), 100) and not draws_from_all(P(temperature=0.8, top_k=5), 100)
    assert not draws_from_all(P(temperature=0.8, top_p=0.9), 100)
    assert not draws_from_all(P(temperature=1.0000000001e-5), 100)           # float32: the limit itself, greedy in the kernel
    assert draws_from_all(P(temperature=0.8, top_p=0.999999999), 100)        # float32: one, no filter in the kernel


def plain_generate(name, prompt, params, eos=()):
    """Tokens of one request chosen the plain way: the whole sequence through the plain model for every token, then
    the reference's order of hard controls, penalties and the draw (rust/engine/src/sampling.rs:220-229, :252-274,
    cuda/sampling.cu)."""
    cfg = tc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    seq = list(prompt)
    for draw in range(params.max_tokens):
        row = plain_llama.forward(cfg, w64, seq)[-1].astype(np.float32)
        row = plain_llama.apply_generation_controls(row, params.min_tokens, len(seq) - len(prompt), eos, params.stop_token_ids,
                                                    params.allowed_token_ids, params.bad_word_ids, seq)
        row = plain_llama.apply_penalties(row, seq, params.repetition_penalty, params.presence_penalty, params.frequency_penalty,
                                          params.repeat_last_n, params.logit_bias)
        token = plain_llama.device_sample(row, params.temperature, params.top_k, params.top_p, params.seed or 0, draw, params.min_p)
        seq.append(token)
        if params.stops_on(token, eos):
            break
    return seq[len(prompt):]


@pytest.mark.parametrize("ahead", [False, True])
def test_penalties_biases_min_tokens_and_min_p_match_the_plain_order(ahead):
    """Requests that ask for what else the reference samples with: penalties on the tokens seen (prompt and
    generated, all of them or a window), biases, end and stop ids blocked for the first tokens, min-p; beside a
    request that asks for nothing.  With steps launched ahead the newest token of a request is counted on the device."""
    plain = SamplingParams(max_tokens=12)
    free = plain_generate("A", PROMPTS_A[1], plain)
    loops = SamplingParams(max_tokens=12, repetition_penalty=1.6, presence_penalty=0.4, frequency_penalty=0.3)
    window = SamplingParams(max_tokens=12, repetition_penalty=1.3, frequency_penalty=0.5, repeat_last_n=3)
    eos = (free[0], free[1])
    held = SamplingParams(max_tokens=8, min_tokens=5, stop_token_ids=(free[2],), logit_bias=((free[3], 4.0), (7, -2.0)))
    drawn = SamplingParams(max_tokens=10, temperature=0.9, top_k=30, min_p=0.08, top_p=0.9, seed=77, presence_penalty=0.6)
    cases = [("loops", PROMPTS_A[1], loops), ("window", PROMPTS_A[2], window), ("held", PROMPTS_A[1], held),
             ("drawn", PROMPTS_A[0], drawn), ("plain", PROMPTS_A[1], plain)]
    engine = make_engine(ahead=ahead, eos_token_ids=eos)
    for name, prompt, params in cases:
        engine.add_request(name, prompt, params)
    got = {name: [] for name, _, _ in cases}
    while engine.has_unfinished():
        for ev in engine.step():
            got[ev.request_id].append(ev.token_id)
    for name, prompt, params in cases:
        assert got[name] == plain_generate("A", prompt, params, eos), name
    assert got["loops"] != free and got["window"] != free            # the penalties do change the tokens
    assert len(got["held"]) >= 5 and not set(got["held"][:5]) & (set(eos) | {free[2]})
    assert got["plain"] == free[:1]                                  # the first token the model gives is an end id here
    engine.runner.cache.check_invariants()


def test_sampling_params_refuse_what_makes_no_sense():
    for bad in (dict(min_p=1.5), dict(min_p=-0.1), dict(repetition_penalty=0.0), dict(min_tokens=-1),
                dict(logit_bias=((3, 1.0), (3, 2.0))), dict(logit_bias=((-1, 1.0),))):
        with pytest.raises(ValueError):
            SamplingParams(**bad)
    p = SamplingParams(presence_penalty=0.5, min_tokens=2)
    assert p.penalizes and p.adjusts_logits(0) and SamplingParams(min_tokens=2).adjusts_logits(1)
    assert not SamplingParams(min_tokens=2).adjusts_logits(2) and not SamplingParams(repetition_penalty=1.000001).penalizes


@pytest.mark.parametrize("ahead", [False, True])
def test_priority_policy_lets_a_better_request_overtake(ahead):
    """One slot: a request of better priority that arrives later takes it, the one that ran waits and later runs its
    prompt and what it had generated again; both end with the tokens they would have had alone."""
    engine = make_engine(max_seqs=1, scheduling_policy="priority", ahead=ahead)
    engine.add_request("low", PROMPTS_A[1], SamplingParams(max_tokens=8, priority=5))
    events = []
    for _ in range(4):
        events += engine.step()
    engine.add_request("high", PROMPTS_A[0], SamplingParams(max_tokens=4, priority=0))
    while engine.has_unfinished():
        events += engine.step()
    tokens = {name: [e.token_id for e in events if e.request_id == name] for name in ("low", "high")}
    assert tokens == {"low": plain_greedy("A", PROMPTS_A[1], 8), "high": plain_greedy("A", PROMPTS_A[0], 4)}
    finished = [e.request_id for e in events if e.finished]
    assert finished == ["high", "low"] and engine.stats.preemptions == 1
    engine.runner.cache.check_invariants()


# ---- prefix cache --------------------------------------------------------------------------------

@pytest.mark.parametrize("ahead", [False, True])
def test_requests_that_share_a_beginning_compute_it_once_and_say_the_same(ahead):
    common = tc.random_ids(37, 512, 3)
    prompts = [common + tc.random_ids(n, 512, 40 + n) for n in (3, 11, 6)] + [common[:20]]
    greedy = SamplingParams(max_tokens=10)
    want = [make_engine("B", ahead=ahead).generate([p], greedy)[0] for p in prompts]
    engine = make_engine("B", ahead=ahead, prefix_cache=True)
    first = engine.generate(prompts[:1], greedy)            # pages of 8 tokens: 40 + 10 - 1 computed tokens leave 6 full pages
    assert engine.runner.cache.cached_pages() == 6 and engine.stats.prefix_hit_tokens == 0
    rows_before = engine.stats.prefill_rows
    rest = engine.generate(prompts[1:], greedy)
    assert first + rest == want
    # 32 of the 37 common tokens lie in full pages; the prompt that is nothing but a known beginning keeps 16 of its 20
    assert engine.stats.prefix_hit_tokens == 32 + 32 + 16
    assert engine.stats.prefill_rows - rows_before == sum(len(p) for p in prompts[1:]) - 80
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == []
    pool = engine.runner.cache.pools[0]
    held = pool.num_pages - pool.available
    assert engine.clear_prefix_cache() == held > 6
    assert all(p.available == p.num_pages for p in engine.runner.cache.pools)
    # the generated tokens are part of what is known: a prompt that goes on where an answer ended starts behind them
    again = prompts[0] + first[0]
    engine.generate([prompts[0]], greedy)
    hits = engine.stats.prefix_hit_tokens
    engine.generate([again + [5]], SamplingParams(max_tokens=2))
    assert engine.stats.prefix_hit_tokens - hits == 48


def test_few_pages_with_known_prefixes_preempt_and_give_the_same_tokens():
    roomy = make_engine().generate(PROMPTS_A, SamplingParams(max_tokens=16))
    for ahead in (False, True):
        tight = make_engine(num_blocks=5, prefix_cache=True, ahead=ahead)
        assert tight.generate(PROMPTS_A, SamplingParams(max_tokens=16)) == roomy
        assert tight.stats.preemptions >= 1
        tight.runner.cache.check_invariants()
        assert tight.generate(PROMPTS_A, SamplingParams(max_tokens=16)) == roomy       # with what the first round left
        tight.runner.cache.check_invariants()


def test_prefix_cache_is_refused_where_pages_do_not_outlive_their_tokens_and_warm_up_leaves_none():
    with pytest.raises(ValueError, match="keep all keys"):
        make_engine("C", prefix_cache=True)
    engine = make_engine(prefix_cache=True)
    engine.warm_up()
    assert engine.runner.cache.cached_pages() == 0 and engine.stats.prefix_hit_tokens == 0
    assert all(p.available == p.num_pages for p in engine.runner.cache.pools)


# ---- log-probabilities ---------------------------------------------------------------------------

@pytest.mark.parametrize("ahead", [False, True])
def test_events_carry_the_models_own_log_probabilities(ahead):
    """Of every generated token and of the likeliest ones, in the distribution before penalties, temperature and
    filters; a request that did not ask gets none; each request its own number of alternatives."""
    cfg = tc.CONFIGS["A"]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    engine = make_engine("A", ahead=ahead)
    params = [SamplingParams(max_tokens=6, logprobs=3, repetition_penalty=1.8, logit_bias=((5, 4.0),)),
              SamplingParams(max_tokens=6),
              SamplingParams(max_tokens=6, logprobs=0, temperature=0.9, top_k=5, seed=3)]
    for i, (prompt, p) in enumerate(zip(PROMPTS_A, params)):
        engine.add_request(f"r{i}", prompt, p)
    events = {f"r{i}": [] for i in range(3)}
    while engine.has_unfinished():
        for ev in engine.step():
            events[ev.request_id].append(ev)
    assert all(ev.logprob is None and ev.top_logprobs is None for ev in events["r1"])
    for i in (0, 2):
        generated = [ev.token_id for ev in events[f"r{i}"]]
        assert len(generated) == 6
        logits = plain_llama.forward(cfg, w64, PROMPTS_A[i] + generated)
        for k, ev in enumerate(events[f"r{i}"]):
            chosen, alternatives = plain_llama.raw_logprobs(logits[len(PROMPTS_A[i]) - 1 + k], ev.token_id, params[i].logprobs)
            assert abs(ev.logprob - chosen) < 1e-4
            assert [t for t, _ in ev.top_logprobs] == [t for t, _ in alternatives]
            assert all(abs(a - b) < 1e-4 for (_, a), (_, b) in zip(ev.top_logprobs, alternatives))
    assert generated_with_penalty_differs(events["r0"])
    with pytest.raises(ValueError, match="between 0 and 20"):
        SamplingParams(logprobs=21)


@pytest.mark.parametrize("ahead", [False, True])
def test_events_carry_the_log_probabilities_of_the_distribution_drawn_from(ahead):
    """`logprobs_processed`: after penalties, biases, temperature and filters; beside a request that asks for the
    model's own in the same steps."""
    cfg = tc.CONFIGS["A"]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    engine = make_engine("A", ahead=ahead)
    params = [SamplingParams(max_tokens=6, logprobs=3, logprobs_processed=True, repetition_penalty=1.8, logit_bias=((5, 4.0),)),
              SamplingParams(max_tokens=6, logprobs=2),
              SamplingParams(max_tokens=6, logprobs=4, logprobs_processed=True, temperature=0.9, top_k=3, seed=3)]
    for i, (prompt, p) in enumerate(zip(PROMPTS_A, params)):
        engine.add_request(f"r{i}", prompt, p)
    events = {f"r{i}": [] for i in range(3)}
    while engine.has_unfinished():
        for ev in engine.step():
            events[ev.request_id].append(ev)
    for i in range(3):
        generated = [ev.token_id for ev in events[f"r{i}"]]
        logits = plain_llama.forward(cfg, w64, PROMPTS_A[i] + generated)
        for k, ev in enumerate(events[f"r{i}"]):
            row = logits[len(PROMPTS_A[i]) - 1 + k]
            p = params[i]
            if p.logprobs_processed:
                seen = plain_llama.apply_penalties(row, PROMPTS_A[i] + generated[:k], p.repetition_penalty, p.presence_penalty,
                                                   p.frequency_penalty, p.repeat_last_n, p.logit_bias)
                chosen, alternatives = plain_llama.processed_logprobs(seen, ev.token_id, p.logprobs, p.temperature, p.top_k, p.top_p, p.min_p)
            else:
                chosen, alternatives = plain_llama.raw_logprobs(row, ev.token_id, p.logprobs)
            assert abs(ev.logprob - chosen) < 1e-4, (i, k)
            assert [t for t, _ in ev.top_logprobs] == [t for t, _ in alternatives], (i, k)
            assert all(abs(a - b) < 1e-4 for (_, a), (_, b) in zip(ev.top_logprobs, alternatives))
    # greedy with a penalty: a point mass on the token that was taken; top-k 3: three alternatives whatever was asked for
    assert all(ev.logprob == 0.0 and ev.top_logprobs == [(ev.token_id, 0.0)] for ev in events["r0"])
    assert all(len(ev.top_logprobs) == 3 and math.isfinite(ev.logprob) for ev in events["r2"])


def generated_with_penalty_differs(events):
    """The request with a penalty and a bias did not always take the model's likeliest token: what is reported is the
    model's distribution, not the one the token was chosen from."""
    return any(ev.top_logprobs[0][0] != ev.token_id for ev in events)


# ---- allow lists, bad words, timeouts ------------------------------------------------------------

@pytest.mark.parametrize("ahead", [False, True])
def test_allow_lists_and_bad_words_match_the_plain_order(ahead):
    """An allow list keeps every choice inside it; a bad word's last token cannot follow its other tokens, also when the
    newest of them is still on the device (steps launched ahead); a word of one token is blocked always."""
    free = plain_generate("A", PROMPTS_A[1], SamplingParams(max_tokens=10))
    assert len(set(zip(free, free[1:]))) > 3
    # what the free run said becomes forbidden: its second token after its first, its fourth after its second and third,
    # and its fifth token anywhere
    words = ((free[0], free[1]), (free[1], free[2], free[3]), (free[4],), (PROMPTS_A[1][-1], free[0], 9))
    barred = SamplingParams(max_tokens=10, bad_word_ids=words)
    fenced = SamplingParams(max_tokens=10, allowed_token_ids=(3, 200, 17, 90, 91, 92, 5000), temperature=0.8, seed=4)
    both = SamplingParams(max_tokens=10, allowed_token_ids=tuple(range(40, 80)), bad_word_ids=((41,), (50, 51)), repetition_penalty=1.4)
    cases = [("barred", PROMPTS_A[1], barred), ("fenced", PROMPTS_A[2], fenced), ("both", PROMPTS_A[0], both),
             ("plain", PROMPTS_A[1], SamplingParams(max_tokens=10))]
    engine = make_engine("A", ahead=ahead)
    for name, prompt, params in cases:
        engine.add_request(name, prompt, params)
    got = {name: [] for name, _, _ in cases}
    while engine.has_unfinished():
        for ev in engine.step():
            got[ev.request_id].append(ev.token_id)
    for name, prompt, params in cases:
        assert got[name] == plain_generate("A", prompt, params), name
    assert got["plain"] == free and got["barred"] != free
    assert got["barred"][0] == free[0] and got["barred"][1] != free[1] and free[4] not in got["barred"]
    assert set(got["fenced"]) <= {3, 200, 17, 90, 91, 92} and set(got["both"]) <= set(range(40, 80)) - {41}


def test_bad_word_blocks_with_and_without_a_token_on_the_device():
    from fllm_amd.sampling.adjust import bad_word_blocks
    words = [(7,), (1, 2, 3), (2, 4), (9, 9, 9, 9), (5, 1, 2, 8)]
    assert bad_word_blocks(words, [5, 1, 2], 3) == ([7, 3, 4, 8], [])
    assert bad_word_blocks(words, [1, 2], 2) == ([7, 3, 4], [])
    # the newest token is not known: what would follow from each value it may have
    assert bad_word_blocks(words, [5, 1, -1], 2) == ([7], [(2, 3), (2, 4), (2, 8)])
    assert bad_word_blocks(words, [9, 9, -1], 2) == ([7], [(2, 4), (9, 9)])
    assert bad_word_blocks(words, [-1], 0) == ([7], [(2, 4)])
    with pytest.raises(ValueError, match="at least one"):
        SamplingParams(bad_word_ids=((),))
    with pytest.raises(ValueError, match="nonnegative"):
        SamplingParams(allowed_token_ids=(-1,))


def test_requests_are_given_up_when_their_time_is_over(monkeypatch):
    """Waiting counts; the pages go back; the other requests go on (rust/engine/src/runtime.rs:1222-1232)."""
    import fllm_amd.engine.engine as module
    now = [100.0]
    monkeypatch.setattr(module.time, "monotonic", lambda: now[0])
    engine = make_engine("A", max_seqs=1)
    engine.add_request("slow", PROMPTS_A[0], SamplingParams(max_tokens=30, timeout_secs=5.0))
    engine.add_request("waits", PROMPTS_A[1], SamplingParams(max_tokens=4, timeout_secs=2.0))
    engine.add_request("patient", PROMPTS_A[1], SamplingParams(max_tokens=4))
    events = engine.step() + engine.step()
    now[0] += 3.0                                   # the waiting request's time is over before it ever ran
    events += engine.step()
    assert [(e.request_id, e.token_id, e.finish_reason) for e in events if e.finished] == [("waits", -1, "timeout")]
    now[0] += 3.0
    assert engine.expire_requests() == ["slow"]
    engine.runner.cache.check_invariants()
    rest = []
    while engine.has_unfinished():
        rest += engine.step()
    assert [e.token_id for e in rest if e.request_id == "patient"] == plain_greedy("A", PROMPTS_A[1], 4)
    assert not any(e.request_id == "slow" for e in rest)
    assert all(p.available == p.num_pages for p in engine.runner.cache.pools)
    with pytest.raises(ValueError, match="positive"):
        SamplingParams(timeout_secs=0.0)


# ---- several answers to a prompt -----------------------------------------------------------------

@pytest.mark.parametrize("ahead", [False, True])
@pytest.mark.parametrize("prefix_cache", [False, True])
def test_several_answers_share_the_prompt_and_draw_for_themselves(ahead, prefix_cache):
    """n answers: the first computes the prompt, the others start behind its full pages (pages of 8 tokens, a prompt
    of 40 and one of 21: 32 and 16 tokens each) and draw with seeds of their own; each is what a request of its own
    with that seed gives.  Greedy answers are all the same."""
    prompt = tc.random_ids(40, 512, 21)
    other = tc.random_ids(21, 512, 22)
    params = SamplingParams(max_tokens=8, temperature=0.9, top_k=20, seed=11, n=3)
    engine = make_engine("B", ahead=ahead, prefix_cache=prefix_cache, max_seqs=8)
    answers, greedy = engine.generate([prompt, other], [params, SamplingParams(max_tokens=5, n=2)])
    assert len(answers) == 3 and len({tuple(a) for a in answers}) == 3 and greedy[0] == greedy[1] and len(greedy[0]) == 5
    alone = make_engine("B", ahead=ahead)
    from dataclasses import replace
    assert answers == [alone.generate([prompt], replace(params.for_choice(k), n=1))[0] for k in range(3)]
    assert greedy[0] == plain_greedy_b(other, 5)
    # the prompt rows that were computed: the whole prompts once, and for every further answer what lies behind the full pages
    assert engine.stats.prefill_rows == 40 + 2 * 8 + 21 + 5
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == [] and not engine.has_unfinished()
    with pytest.raises(ValueError, match="between 1 and 16"):
        SamplingParams(n=17)


def plain_greedy_b(prompt, count):
    cfg = tc.CONFIGS["B"]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    seq = list(prompt)
    for _ in range(count):
        seq.append(plain_llama.greedy(plain_llama.forward(cfg, w64, seq)[-1]))
    return seq[len(prompt):]


def test_answers_end_one_by_one_and_abort_together():
    engine = make_engine("A", max_seqs=4)
    engine.add_request("r", PROMPTS_A[1], SamplingParams(max_tokens=6, temperature=1.0, seed=2, n=3))
    events = []
    for _ in range(4):
        events += engine.step()
    assert {e.choice for e in events} == {0, 1, 2}
    engine.abort_request("r")
    assert not engine.scheduler.has_work() and engine.runner.cache.requests() == []
    while engine.has_unfinished():
        assert engine.step() == []
    engine.add_request("r", PROMPTS_A[0], SamplingParams(max_tokens=3, n=2))
    engine.abort_request("r")                       # before the first answer's prompt ran: the others never begin
    assert not engine.has_unfinished() and engine._followers == {}
    finished = []
    engine.add_request("q", PROMPTS_A[0], SamplingParams(max_tokens=3, temperature=1.0, seed=1, n=2))
    while engine.has_unfinished():
        finished += [(e.choice, e.finish_reason) for e in engine.step() if e.finished]
    assert sorted(finished) == [(0, "length"), (1, "length")]
    engine.runner.cache.check_invariants()
