"""Random requests with random sampling options through the engine on the CPU (the plain kernels of
tests/reference_ops.py in place of the HIP library): whatever the scheduling (steps that wait or are launched ahead,
room for everything or so few pages that requests are preempted, prefixes kept or not, first come or by priority),
every answer of every request must be the same tokens, and the cache manager's books must balance at the end."""
import random

import pytest

import tiny_configs as tc
from reference_ops import ReferenceOps
from fllm_amd import Engine, SamplingParams


def random_params(rng, vocab):
    kw = dict(max_tokens=rng.randint(2, 14), priority=rng.randint(-2, 2))
    chance = rng.random
    if chance() < 0.6:
        kw.update(temperature=rng.choice([0.3, 0.8, 1.0, 2.0]), seed=rng.randint(0, 99))
    if chance() < 0.3:
        kw["top_k"] = rng.choice([1, 5, 40, vocab])
    if chance() < 0.3:
        kw["top_p"] = rng.choice([0.1, 0.7, 0.95])
    if chance() < 0.3:
        kw["min_p"] = rng.choice([0.01, 0.1, 0.5])
    if chance() < 0.3:
        kw["repetition_penalty"] = rng.choice([0.8, 1.2, 2.0])
    if chance() < 0.3:
        kw["presence_penalty"] = rng.choice([-0.5, 0.5])
    if chance() < 0.3:
        kw["frequency_penalty"] = rng.choice([0.2, 1.0])
    if chance() < 0.3:
        kw["repeat_last_n"] = rng.choice([0, 1, 4, 50])
    if chance() < 0.3:
        kw["min_tokens"] = rng.randint(1, 6)
    if chance() < 0.3:
        kw["logit_bias"] = tuple((t, rng.uniform(-3, 3)) for t in rng.sample(range(vocab), 3))
    if chance() < 0.3:
        kw["stop_token_ids"] = tuple(rng.sample(range(vocab), 4))
    if chance() < 0.2:
        kw["allowed_token_ids"] = tuple(rng.sample(range(vocab), rng.choice([2, 30])))
    if chance() < 0.3:
        kw["bad_word_ids"] = tuple(tuple(rng.randrange(12) for _ in range(rng.randint(1, 3))) for _ in range(6))
    if chance() < 0.2:
        kw["logprobs"] = rng.choice([0, 3])
    if chance() < 0.25:
        kw["n"] = rng.randint(2, 3)
    return SamplingParams(**kw)


def run(cfg_name, requests, eos, device="cpu", **options):
    cfg = tc.CONFIGS[cfg_name]
    if device == "cpu":
        options["ops"] = ReferenceOps()
    engine = Engine(config=cfg, seed=1, dtype="float32", device=device, ctx=cfg["max_position_embeddings"], max_seqs=4,
                    block_size=tc.PAGE_SIZES[cfg_name], eos_token_ids=eos, **options)
    for rid, prompt, params in requests:
        engine.add_request(rid, prompt, params)
    got = {}
    while engine.has_unfinished():
        for ev in engine.step():
            got.setdefault((ev.request_id, ev.choice), []).append(ev.token_id)
            assert (ev.logprob is not None) == (dict((r, p) for r, _, p in requests)[ev.request_id].logprobs is not None)
    engine.runner.cache.check_invariants()
    engine.clear_prefix_cache()
    assert engine.runner.cache.requests() == [] and all(p.available == p.num_pages for p in engine.runner.cache.pools)
    return got, engine.stats


@pytest.mark.parametrize("trial", range(10))
def test_tokens_do_not_depend_on_the_scheduling(trial):
    scheduling_does_not_matter(trial, "cpu")


@pytest.mark.gpu
@pytest.mark.parametrize("trial", range(100, 106))
def test_tokens_do_not_depend_on_the_scheduling_on_the_device(trial):
    """The same in true 32-bit on the device, through the HIP kernels, decode graphs and the device's sampler."""
    scheduling_does_not_matter(trial, "cuda:0")


def scheduling_does_not_matter(trial, device):
    rng = random.Random(900 + trial)
    name = rng.choice(["A", "B"])
    vocab = tc.CONFIGS[name]["vocab_size"]
    common = tc.random_ids(rng.randint(8, 40), vocab, trial)            # some requests begin alike
    requests = []
    for i in range(rng.randint(2, 6)):
        own = [t % 12 if rng.random() < 0.3 else t for t in tc.random_ids(rng.randint(1, 30), vocab, trial * 10 + i)]
        requests.append((f"r{i}", (common if rng.random() < 0.5 else []) + own, random_params(rng, vocab)))
    eos = tuple(rng.sample(range(vocab), 3))
    budget = rng.choice([8, 32])
    want, _ = run(name, requests, eos, device, ahead=False, num_blocks=128, max_batched_tokens=budget)
    assert len(want) == sum(p.n for _, _, p in requests) and all(want.values())
    ahead, _ = run(name, requests, eos, device, ahead=True, num_blocks=128, max_batched_tokens=budget)
    assert ahead == want
    longest = max(len(prompt) + p.max_tokens for _, prompt, p in requests)
    pages = -(-longest // tc.PAGE_SIZES[name]) + rng.choice([1, 3])     # room for the longest request and little more
    tight, stats = run(name, requests, eos, device, ahead=True, num_blocks=pages, max_batched_tokens=budget,
                       prefix_cache=rng.random() < 0.5, scheduling_policy=rng.choice(["fcfs", "priority"]))
    assert tight == want, stats
