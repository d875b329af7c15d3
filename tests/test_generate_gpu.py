"""Greedy and sampled generation through the entry points (Engine.generate, the command line)
on the GPU, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_llama
import tiny_configs as tc
from fllm_amd import Engine, SamplingParams
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights import random_tensors, write_random_model

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROMPT_LENGTHS = {"A": (5, 17, 31), "B": (1, 9, 40, 100), "E": (5, 50, 90)}


def make_engine(name, dtype, **kw):
    opts = dict(dtype=dtype, ctx=tc.CONFIGS[name]["max_position_embeddings"], max_seqs=4, max_batched_tokens=32,
                block_size=tc.PAGE_SIZES[name], num_blocks=128)
    opts.update(kw)
    return Engine(config=tc.CONFIGS[name], seed=1, **opts)


def check_greedy(name, dtype, prompts, outputs):
    """Every generated token is the plain implementation's choice given the tokens before it, or,
    where two logits nearly tie, one of the two."""
    cfg = tc.CONFIGS[name]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    tol = 3e-6 if dtype == "float32" else 1.5e-2         # the tolerances of the replay tests
    for prompt, out in zip(prompts, outputs):
        seq = list(prompt)
        logits = plain_llama.forward(cfg, w64, seq + list(out))
        for i, token in enumerate(out):
            row = logits[len(prompt) - 1 + i]
            best = plain_llama.greedy(row)
            assert token == best or row[best] - row[token] <= 2 * tol * np.abs(row).max(), \
                f"{name} {dtype}: token {i} is {token}, the plain implementation takes {best}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_greedy_generation(name, dtype):
    """E decodes far past its window of 40: pages behind the window go back while the request runs."""
    prompts = [tc.random_ids(n, tc.CONFIGS[name]["vocab_size"], 10 + n) for n in PROMPT_LENGTHS[name]]
    count = {"A": 16, "B": 24, "E": 70}[name]
    engine = make_engine(name, dtype)
    outputs = engine.generate(prompts, SamplingParams(max_tokens=count))
    assert all(len(o) == count for o in outputs)
    check_greedy(name, dtype, prompts, outputs)
    assert engine.runner.graph_replays > 0
    engine.runner.cache.check_invariants()


def test_alone_batched_and_preempted_give_the_same_tokens():
    prompts = [tc.random_ids(n, 256, 10 + n) for n in PROMPT_LENGTHS["A"]]
    params = SamplingParams(max_tokens=16)
    together = make_engine("A", "float32").generate(prompts, params)
    alone = [make_engine("A", "float32").generate([p], params)[0] for p in prompts]
    assert together == alone
    tight = make_engine("A", "float32", num_blocks=5)
    assert tight.generate(prompts, params) == together and tight.stats.preemptions >= 1
    eager = make_engine("A", "float32")
    eager.runner.use_graphs = False
    assert eager.generate(prompts, params) == together


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sampled_generation_is_reproducible(dtype):
    """Config B's workload: chunked prefill (portions of 32) mixed with decode, 24 tokens at
    temperature 0.8 from a fixed seed."""
    prompts = [tc.random_ids(n, 512, 20 + n) for n in PROMPT_LENGTHS["B"]]
    params = SamplingParams(max_tokens=24, temperature=0.8, seed=4242)
    a = make_engine("B", dtype).generate(prompts, params)
    b = make_engine("B", dtype).generate(prompts, params)
    assert a == b and all(len(o) == 24 for o in a)
    if dtype == "float32":
        alone = [make_engine("B", dtype).generate([p], params)[0] for p in prompts]
        assert alone == a                                    # the neighbours in the batch do not matter
        # every token is what the plain sampler draws from the plain logits (near-ties aside)
        cfg = tc.TINY_B
        _, spec = model_spec_from_config(cfg)
        w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
        seq = list(prompts[1])
        agree = 0
        for draw, token in enumerate(a[1]):
            logits = plain_llama.forward(cfg, w64, seq)[-1]
            agree += token == plain_llama.device_sample(logits, 0.8, 0, 1.0, 4242, draw)
            seq.append(token)
        # one of the 24 may differ: the draw is the largest of logit / T + noise, and where the two largest of those
        # lie closer together than the engine's float32 logits are to the plain float64 ones (about 1e-6 of the largest
        # logit) either may come out; from then on the comparison follows the engine's token, so one miss stays one
        assert agree >= 23, f"{24 - agree} of 24 sampled tokens are not what the plain sampler draws from the plain logits"
    assert make_engine("B", dtype).generate(prompts, SamplingParams(max_tokens=24, temperature=0.8, seed=1)) != a


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_launched_ahead_give_the_same_tokens(dtype):
    """With `ahead` the device takes a decode row's token from the output of the step before; the tokens are the
    same as when every step waits for the last: greedy and sampled, graphs and eager steps, few pages."""
    prompts = [tc.random_ids(n, 512, 20 + n) for n in PROMPT_LENGTHS["B"]]
    for params in (SamplingParams(max_tokens=24), SamplingParams(max_tokens=24, temperature=0.8, top_p=0.9, seed=7)):
        want = make_engine("B", dtype, ahead=False).generate(prompts, params)
        ahead = make_engine("B", dtype, ahead=True)
        assert ahead.generate(prompts, params) == want
        assert ahead.runner.graph_replays > 0
        ahead.runner.cache.check_invariants()
        eager = make_engine("B", dtype, ahead=True)
        eager.runner.use_graphs = False
        assert eager.generate(prompts, params) == want
    tight = make_engine("B", dtype, ahead=True, num_blocks=26)
    assert tight.generate(prompts, SamplingParams(max_tokens=24)) == make_engine("B", dtype, ahead=False).generate(prompts, SamplingParams(max_tokens=24))
    assert tight.stats.preemptions >= 1
    tight.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_penalties_biases_min_tokens_and_min_p(dtype):
    """What else the reference samples with, on the device: penalties over the tokens seen (all of them, or a
    window), biases, end and stop ids blocked for the first tokens, min-p.  Steps launched ahead (the newest token of
    a request is counted from the device's copy) give the tokens of steps that wait; in float32 they are the plain
    order's tokens, computed from the plain model's logits."""
    cfg = tc.CONFIGS["A"]
    prompts = [tc.random_ids(n, cfg["vocab_size"], 10 + n) for n in PROMPT_LENGTHS["A"]]
    free = make_engine("A", dtype).generate([prompts[1]], SamplingParams(max_tokens=12))[0]
    eos = (free[0], free[1])
    cases = [("loops", prompts[1], SamplingParams(max_tokens=12, repetition_penalty=1.6, presence_penalty=0.4, frequency_penalty=0.3)),
             ("window", prompts[2], SamplingParams(max_tokens=12, repetition_penalty=1.3, frequency_penalty=0.5, repeat_last_n=3)),
             ("held", prompts[1], SamplingParams(max_tokens=8, min_tokens=5, stop_token_ids=(free[2],), logit_bias=((free[3], 4.0), (7, -2.0)))),
             ("drawn", prompts[0], SamplingParams(max_tokens=10, temperature=0.9, top_k=30, min_p=0.08, top_p=0.9, seed=77, presence_penalty=0.6)),
             ("barred", prompts[1], SamplingParams(max_tokens=12, bad_word_ids=((free[4], free[5]), (free[5], free[6], free[7]), (free[8],)))),
             ("fenced", prompts[2], SamplingParams(max_tokens=10, allowed_token_ids=tuple(range(30, 90)), bad_word_ids=((31,), (40, 41)),
                                                   temperature=0.7, seed=3)),
             ("plain", prompts[1], SamplingParams(max_tokens=12))]

    def run(ahead, graphs=True):
        engine = make_engine("A", dtype, ahead=ahead, eos_token_ids=eos, max_seqs=8)
        engine.runner.use_graphs = graphs
        for name, prompt, params in cases:
            engine.add_request(name, prompt, params)
        got = {name: [] for name, _, _ in cases}
        while engine.has_unfinished():
            for ev in engine.step():
                got[ev.request_id].append(ev.token_id)
        engine.runner.cache.check_invariants()
        return got

    waited = run(False)
    assert run(True) == waited and run(True, graphs=False) == waited
    assert waited["loops"] != free and waited["window"] != free and waited["plain"] == free[:1]
    assert len(waited["held"]) >= 5 and not set(waited["held"][:5]) & (set(eos) | {free[2]})
    assert set(waited["fenced"]) <= set(range(30, 90)) - {31} and free[8] not in waited["barred"]
    if dtype == "float32":
        _, spec = model_spec_from_config(cfg)
        w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
        for name, prompt, params in cases:
            seq, agree = list(prompt), 0
            for draw, token in enumerate(waited[name]):
                row = plain_llama.forward(cfg, w64, seq)[-1].astype(np.float32)
                row = plain_llama.apply_generation_controls(row, params.min_tokens, draw, eos, params.stop_token_ids,
                                                            params.allowed_token_ids, params.bad_word_ids, seq)
                row = plain_llama.apply_penalties(row, seq, params.repetition_penalty, params.presence_penalty,
                                                  params.frequency_penalty, params.repeat_last_n, params.logit_bias)
                agree += token == plain_llama.device_sample(row, params.temperature, params.top_k, params.top_p, params.seed or 0,
                                                            draw, params.min_p)
                seq.append(token)
            assert agree >= len(waited[name]) - 1, name          # a near-tie may fall the other way


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_known_prefixes_are_taken_over_and_given_up(name, dtype):
    """Requests that begin alike start behind the pages of the first; with few pages those are given up and used
    again for other tokens, and a later request with the same beginning computes it anew."""
    vocab = tc.CONFIGS[name]["vocab_size"]
    page = tc.PAGE_SIZES[name]
    common = tc.random_ids(5 * page + 3, vocab, 77)
    prompts = [common + tc.random_ids(n, vocab, 30 + n) for n in (4, 9, 2 * page)] + [common[:3 * page]]
    params = SamplingParams(max_tokens=12)
    engine = make_engine(name, dtype, prefix_cache=True)
    outputs = engine.generate(prompts[:1], params) + engine.generate(prompts[1:], params)
    check_greedy(name, dtype, prompts, outputs)
    assert engine.stats.prefix_hit_tokens == (5 + 5 + 2) * page
    engine.runner.cache.check_invariants()
    # room for one request and a little more: every request finds some of the first one's pages gone
    others = [tc.random_ids(6 * page, vocab, 90 + i) for i in range(3)]
    tight = make_engine(name, dtype, prefix_cache=True, num_blocks=9, max_seqs=2)
    order = [prompts[0], others[0], prompts[1], others[1], others[2], prompts[2], prompts[0]]
    outputs = [tight.generate([p], params)[0] for p in order]
    check_greedy(name, dtype, order, outputs)
    if dtype == "float32":
        assert outputs[6] == outputs[0]
    assert tight.runner.cache.cached_pages() <= 9 and tight.stats.prefix_hit_tokens > 0
    tight.runner.cache.check_invariants()
    assert tight.clear_prefix_cache() > 0 and all(p.available == p.num_pages for p in tight.runner.cache.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_log_probabilities_come_with_the_tokens(dtype):
    """The model's own distribution (before the penalty that steers the choice), for the chosen token and the
    likeliest ones, through steps launched ahead and decode graphs."""
    cfg = tc.CONFIGS["B"]
    _, spec = model_spec_from_config(cfg)
    w64 = tc.to_float64(random_tensors(spec, 1, torch.float32))
    prompts = [tc.random_ids(n, cfg["vocab_size"], 10 + n) for n in (9, 40)]
    params = [SamplingParams(max_tokens=12, logprobs=4, repetition_penalty=1.5), SamplingParams(max_tokens=12, logprobs=20, temperature=0.8, seed=7)]
    engine = make_engine("B", dtype)
    for i, (prompt, p) in enumerate(zip(prompts, params)):
        engine.add_request(f"r{i}", prompt, p)
    events = {"r0": [], "r1": []}
    while engine.has_unfinished():
        for ev in engine.step():
            events[ev.request_id].append(ev)
    tol = 3e-6 if dtype == "float32" else 1.5e-2
    for i, prompt in enumerate(prompts):
        generated = [ev.token_id for ev in events[f"r{i}"]]
        logits = plain_llama.forward(cfg, w64, prompt + generated)
        for k, ev in enumerate(events[f"r{i}"]):
            row = logits[len(prompt) - 1 + k]
            want = torch.log_softmax(torch.from_numpy(np.asarray(row, dtype=np.float64)), 0)
            allowed = 4 * tol * np.abs(row).max() + 1e-5
            assert abs(ev.logprob - float(want[ev.token_id])) <= allowed
            assert len(ev.top_logprobs) == params[i].logprobs
            values = [v for _, v in ev.top_logprobs]
            assert values == sorted(values, reverse=True) and len({t for t, _ in ev.top_logprobs}) == len(values)
            assert all(abs(v - float(want[t])) <= allowed for t, v in ev.top_logprobs)
            assert values[0] >= float(want.max()) - allowed and values[-1] >= float(torch.sort(want).values[-len(values)]) - allowed
    assert engine.runner.graph_replays > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_several_answers_to_a_prompt(dtype):
    """The further answers start on the first one's full pages (which nobody writes again) and draw with seeds of
    their own: in float32 each is the answer of a request of its own with that seed; the greedy ones agree with the
    plain implementation."""
    from dataclasses import replace
    vocab = tc.CONFIGS["B"]["vocab_size"]
    prompt, other = tc.random_ids(100, vocab, 5), tc.random_ids(37, vocab, 6)
    drawn = SamplingParams(max_tokens=12, temperature=0.8, top_p=0.95, seed=9, n=4)
    engine = make_engine("B", dtype, max_seqs=8)
    answers, greedy = engine.generate([prompt, other], [drawn, SamplingParams(max_tokens=12, n=3)])
    assert len({tuple(a) for a in answers}) == 4 and all(len(a) == 12 for a in answers)
    check_greedy("B", dtype, [other] * 3, greedy)
    assert engine.stats.prefill_rows == 100 + 3 * 4 + 37 + 2 * 5          # pages of 8 tokens
    if dtype == "float32":
        alone = make_engine("B", dtype)
        assert answers == [alone.generate([prompt], replace(drawn.for_choice(k), n=1))[0] for k in range(4)]
        assert greedy[0] == greedy[1] == greedy[2]
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == []


def test_no_garbage_collection_while_a_graph_is_captured():
    """Engines that went before leave cycles behind; their collection frees graphs and pinned buffers through the
    HIP runtime, which must not happen while a stream is capturing: the collector is off for the capture's
    length and on again after it."""
    import gc
    prompts = [tc.random_ids(n, 512, 40 + n) for n in PROMPT_LENGTHS["B"]]
    params = SamplingParams(max_tokens=6)
    want = make_engine("B", "bfloat16", ahead=True).generate(prompts, params)     # left behind for the collector
    engine = make_engine("B", "bfloat16", ahead=True)
    seen = []
    forward = engine.runner.model.forward

    def watched(ctx):
        seen.append((torch.cuda.is_current_stream_capturing(), gc.isenabled()))
        return forward(ctx)

    engine.runner.model.forward = watched
    assert gc.isenabled()
    assert engine.generate(prompts, params) == want
    assert gc.isenabled()
    assert any(capturing for capturing, _ in seen)
    assert all(not collecting for capturing, collecting in seen if capturing)
    assert any(collecting for capturing, collecting in seen if not capturing)


def test_command_line(tmp_path):
    folder = str(tmp_path / "model")
    write_random_model(folder, tc.TINY_A, seed=1, dtype="float32")
    prompt = tc.random_ids(9, 256, 3)
    cmd = [sys.executable, "-m", "fllm_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8",
           "--dtype", "float32", "--kv-blocks", "16", "--max-seqs", "2"]
    proc = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr
    record = json.loads(proc.stdout.strip().splitlines()[0])
    assert record["finish_reason"] == "length" and len(record["token_ids"]) == 8
    check_greedy("A", "float32", [prompt], [record["token_ids"]])
    assert "forward_calls=" in proc.stderr
    # the further sampling options, by the reference's flag names: the tokens of the same options through the entry point
    first = record["token_ids"]
    flags = ["--repeat-penalty", "1.5", "--presence-penalty", "0.3", "--frequency-penalty", "0.2", "--repeat-last-n", "6",
             "--min-tokens", "3", "--stop-token-ids", str(first[0]), "--logit-bias", f"{first[1]}:-5,3:0.5", "--min-p", "0.1",
             "--temperature", "0.7", "--seed", "5", "--prefix-cache", "--logprobs", "2", "--bad-words-ids", f"{first[2]},{first[3]}",
             "--allowed-token-ids", ",".join(str(t) for t in range(256) if t != first[4]), "--timeout", "60", "--n", "2"]
    proc = subprocess.run(cmd + flags, cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr
    assert "prefix_hit_tokens=0" in proc.stderr
    record = json.loads(proc.stdout.strip().splitlines()[0])
    assert len(record["logprobs"]) == len(record["token_ids"]) and all(len(e["top"]) == 2 and e["logprob"] <= 0 for e in record["logprobs"])
    second = json.loads(proc.stdout.strip().splitlines()[1])
    assert record["choice"] == 0 and second["choice"] == 1 and second["token_ids"] != record["token_ids"]
    record = json.loads(proc.stdout.strip().splitlines()[0])
    params = SamplingParams(max_tokens=8, temperature=0.7, seed=5, min_p=0.1, repetition_penalty=1.5, presence_penalty=0.3,
                            frequency_penalty=0.2, repeat_last_n=6, min_tokens=3, stop_token_ids=(first[0],),
                            logit_bias=((first[1], -5.0), (3, 0.5)), bad_word_ids=((first[2], first[3]),),
                            allowed_token_ids=tuple(t for t in range(256) if t != first[4]))
    engine = Engine(folder, dtype="float32", num_blocks=16, max_seqs=2)
    assert record["token_ids"] == engine.generate([prompt], params)[0] and first[0] not in record["token_ids"][:3]
    # sampling defaults and end-of-sequence ids that ship with the model: flags that are left out take them, `vllm` ignores them
    with open(os.path.join(folder, "generation_config.json"), "w") as fh:
        json.dump({"temperature": 0.9, "top_k": 12, "repetition_penalty": 1.3, "eos_token_id": [first[5]]}, fh)
    config = json.load(open(os.path.join(folder, "config.json")))
    config.pop("eos_token_id", None)
    with open(os.path.join(folder, "config.json"), "w") as fh:
        json.dump(config, fh)
    proc = subprocess.run(cmd + ["--seed", "8", "--top-k", "20"], cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0 and "sampling defaults from" in proc.stderr, proc.stderr
    engine = Engine(folder, dtype="float32", num_blocks=16, max_seqs=2)
    assert engine.eos_token_ids == (first[5],)
    want = engine.generate([prompt], SamplingParams(max_tokens=8, temperature=0.9, top_k=20, repetition_penalty=1.3, seed=8))[0]
    assert json.loads(proc.stdout.strip().splitlines()[0])["token_ids"] == want
    proc = subprocess.run(cmd + ["--generation-config", "vllm"], cwd=ROOT, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr
    assert json.loads(proc.stdout.strip().splitlines()[0])["token_ids"] == engine.generate([prompt], SamplingParams(max_tokens=8))[0]


@pytest.mark.parametrize("budget,prompt_len", [(512, 512), (2, 40)])
def test_single_token_portion_with_pages_reserved_ahead(budget, prompt_len):
    """A prompt's last portion (or, under a tiny budget, every portion) can be one token: the step is then all
    single tokens and runs as a graph, while the request's block table already holds the pages of the whole
    prompt plus one, more entries than the graph's table rows are wide.  The tokens are those of a run that
    cuts nothing."""
    first = tc.random_ids(40, 384, 1)
    second = tc.random_ids(prompt_len, 384, 2)
    params = SamplingParams(max_tokens=12)
    base = dict(ctx=1024, max_seqs=4, block_size=16, num_blocks=160, decode_first=True)
    want = [make_engine("D", "float32", max_batched_tokens=1024, **base).generate([p], params)[0] for p in (first, second)]
    engine = make_engine("D", "float32", max_batched_tokens=budget, **base)
    engine.add_request("first", first, params)
    outputs = {"first": [], "second": []}
    for _ in range(3 if budget > 2 else 22):          # "first" is decoding when "second" arrives
        for ev in engine.step():
            outputs[ev.request_id].append(ev.token_id)
    engine.add_request("second", second, params)
    while engine.has_unfinished():
        for ev in engine.step():
            outputs[ev.request_id].append(ev.token_id)
    assert [outputs["first"], outputs["second"]] == want
    assert engine.runner.graph_replays > 0
    engine.runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_ahead_stop_token_with_pages_that_change_hands(dtype):
    """Steps launched ahead, a request that stops at a token, and so few pages that the next request can only start
    on the pages the stopped one gives back: when the stop token reaches the host, one more row of that request is
    already in flight; it is dropped, its pages go to the waiting request, and that request's tokens are what it
    generates alone."""
    import trace_tools as tt
    stopper, waiter = tc.random_ids(17, 256, 31), tc.random_ids(31, 256, 32)
    alone = [make_engine("A", dtype).generate([p], SamplingParams(max_tokens=10))[0] for p in (stopper, waiter)]
    stop_at = 3
    assert alone[0][stop_at] not in alone[0][:stop_at]
    engine = make_engine("A", dtype, ahead=True, num_blocks=3, max_seqs=2)
    handed_out = tt.record_allocations(engine.runner.cache)
    sid = engine.add_request("stopper", stopper, SamplingParams(max_tokens=10, stop_token_ids=(alone[0][stop_at],)))
    engine.add_request("waiter", waiter, SamplingParams(max_tokens=10))
    outputs = {"stopper": [], "waiter": []}
    row_in_flight_at_the_stop = False
    while engine.has_unfinished():
        for ev in engine.step():
            outputs[ev.request_id].append(ev.token_id)
            if ev.request_id == "stopper" and ev.finished:
                assert ev.finish_reason == "stop"
                row_in_flight_at_the_stop = engine._in_flight is not None and sid in engine._in_flight.sampled
                assert not outputs["waiter"], "the waiting request was to start only on the pages given back"
    assert row_in_flight_at_the_stop
    assert outputs["stopper"] == alone[0][:stop_at + 1]
    assert outputs["waiter"] == alone[1]
    assert len(handed_out[0]) > len(set(handed_out[0])), "no page changed hands"
    engine.runner.cache.check_invariants()
    assert engine.runner.cache.requests() == []


def test_warm_up_captures_the_graphs_before_the_first_request():
    """After `warm_up` the decode graphs of every batch size up to `max_seqs`, for short and long contexts, exist; the
    first real requests capture nothing, and their tokens are those of an engine that was not warmed up."""
    prompts = [tc.random_ids(n, 384, 60 + n) for n in (5, 300, 40)]
    params = SamplingParams(max_tokens=12)
    want = make_engine("D", "bfloat16", ctx=1024, num_blocks=256).generate(prompts, params)
    engine = make_engine("D", "bfloat16", ctx=1024, num_blocks=256)
    assert engine.warm_up() > 0
    keys = set(engine.runner._graphs)
    assert {(rows, bound) for rows in (1, 2, 4) for bound in (256, 512, 1024)} <= keys
    assert engine.stats.forward_calls == 0 and engine.runner.cache.requests() == []
    assert engine.generate(prompts, params) == want
    assert set(engine.runner._graphs) == keys, "a graph was captured after the warm-up"
    engine.runner.cache.check_invariants()


def test_layer_check_names_the_layer_that_goes_wrong():
    """Every layer of the first steps runs with the plain kernels and with the serving kernels on the same input.
    Healthy: the two stay within bfloat16 rounding of each other.  With the serving run of one layer's attention
    disturbed, that layer is the first suspect."""
    import io
    prompt = tc.random_ids(40, 384, 77)
    log = io.StringIO()
    healthy = make_engine("D", "bfloat16", ctx=1024, num_blocks=64, max_batched_tokens=64, check_layers=3)
    healthy.layer_check.out = log
    want = make_engine("D", "bfloat16", ctx=1024, num_blocks=64, max_batched_tokens=64).generate([prompt], SamplingParams(max_tokens=6))
    assert healthy.generate([prompt], SamplingParams(max_tokens=6)) == want          # the check changes no token
    reports = healthy.layer_check.reports
    assert len(reports) == 3 * 2 and [r.rows for r in reports] == [40, 40, 1, 1, 1, 1]
    assert all(r.distance is not None and r.distance < 2e-2 and r.bad_values == 0 for r in reports), log.getvalue()
    assert healthy.layer_check.suspects() == [] and healthy.runner.graph_replays > 0   # graphs again once the check is over

    broken = make_engine("D", "bfloat16", ctx=1024, num_blocks=64, max_batched_tokens=64, check_layers=1)
    broken.layer_check.out = log
    ops = broken.runner.rt.ops
    calls = []
    attention = ops.attention

    def disturbed(*args, **kw):
        out = attention(*args, **kw)
        calls.append(1)
        if len(calls) == 4:                   # layer 0 plain, layer 0 serving, layer 1 plain, layer 1 serving
            out.mul_(1.5)
        return out

    ops.attention = disturbed
    try:
        broken.generate([prompt], SamplingParams(max_tokens=1))
    finally:
        del ops.attention
    suspects = broken.layer_check.suspects()
    assert [r.entry for r in suspects] == [1] and "first suspect: step 0, run entry 1" in log.getvalue()
