"""Replays the same requests whole, with the last 32 tokens one by one, in portions of changing
size, and mixed with other requests on so few pages that they are used again, in float32 and in
bfloat16, and compares every logit with the plain implementation."""
import os

import numpy as np
import pytest
import torch

import plain_llama
import tiny_configs as tc
import trace_tools as tt

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 31, 70, 128, 100], "B": [1, 9, 40, 100, 256, 130], "C": [3, 50, 190, 77, 120, 64],
           "D": [700, 3, 130, 1000, 64], "E": [300, 45, 130, 500, 64, 90], "F": [4, 60, 256, 33, 150, 90],
           "G": [2, 48, 160, 49, 100, 70]}
# |engine - plain| <= tol * max|plain logit| ; float32 engine against a float64 reference, and
# bfloat16 (8 bits of mantissa in weights, activations and cache) against the same.  About three times the largest
# error any case here has shown on the MI355X (float32 7.9e-7, bfloat16 6.0e-3; the test session prints them).
TOL = {"float32": 3e-6, "bfloat16": 1.5e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """Model folders written with the safetensors library (not the engine's writer), in bfloat16-exact
    float32 values so that both precisions read the same weights."""
    from safetensors.torch import save_file
    import json
    from fllm_amd.registry import model_spec_from_config
    from fllm_amd.weights import random_tensors
    out = {}
    for name, cfg in tc.CONFIGS.items():
        _, spec = model_spec_from_config(cfg)
        tensors = random_tensors(spec, seed=11 + ord(name), dtype=torch.bfloat16, with_optional=(name == "C"))
        tensors = {k: v.to(torch.float32) for k, v in tensors.items()}
        folder = str(tmp_path_factory.mktemp(f"tiny_{name}"))
        with open(os.path.join(folder, "config.json"), "w") as fh:
            json.dump(cfg, fh)
        save_file(tensors, os.path.join(folder, "model.safetensors"))
        requests = {f"r{i}": tc.random_ids(n, cfg["vocab_size"], 100 * ord(name) + i) for i, n in enumerate(LENGTHS[name])}
        w64 = tc.to_float64(tensors)
        plain = {rid: plain_llama.forward(cfg, w64, toks) for rid, toks in requests.items()}
        out[name] = (folder, cfg, requests, plain)
    return out


def check(got, plain, dtype, what):
    for rid, want in plain.items():
        assert rid in got, f"{what}: request {rid} missing"
        assert got[rid].shape == want.shape, f"{what}: {rid} has shape {got[rid].shape}, expected {want.shape}"
        err = np.abs(got[rid].astype(np.float64) - want)
        scale = np.abs(want).max()
        pos = int(err.max(axis=1).argmax())
        tt.observe(f"replay {what.split()[0]} {dtype}", err.max() / scale)
        assert err.max() <= TOL[dtype] * scale, (f"{what}: request {rid}: max error {err.max():.3e} at position {pos} "
                                                 f"(limit {TOL[dtype] * scale:.3e}); first position over the limit: "
                                                 f"{int(np.argmax(err.max(axis=1) > TOL[dtype] * scale))}")


def make_runner(folder, dtype, page_size, max_tokens, use_graphs=True):
    from fllm_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=8,
                                   use_graphs=use_graphs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G"])
@pytest.mark.parametrize("family", ["whole", "last32", "portions", "mixed"])
def test_replay(models, tmp_path, name, dtype, family):
    folder, cfg, requests, plain = models[name]
    refed = [rid for rid, toks in requests.items() if len(toks) >= 60][:2]
    steps = {"whole": tt.whole, "last32": tt.last_tokens_one_by_one, "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=5, refeed=refed)}[family](requests)
    steps = tt.number(steps)
    max_tokens = tt.live_tokens_bound(steps)
    runner = make_runner(folder, dtype, tc.PAGE_SIZES[name], max_tokens)
    handed_out = tt.record_allocations(runner.cache)
    given_up = {}
    got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path), given_up)
    check(got, plain, dtype, f"{name} {dtype} {family}")
    if family == "mixed":
        # a request that was ended half way and fed again from its first token (as after a preemption) gave the same
        # logits the first time, on other pages and in other company
        assert sorted(given_up) == sorted(refed)
        for rid, feedings in given_up.items():
            for first in feedings:
                assert len(first) >= len(requests[rid]) // 2
                if dtype == "float32":
                    assert np.array_equal(first, got[rid][:len(first)]), f"{rid}: fed again, other logits"
                check({rid: first}, {rid: plain[rid][:len(first)]}, dtype, f"{name} {dtype} given-up")
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools), "pages were lost"
    for pages in handed_out:
        assert len(pages) > len(set(pages)), "the trace was meant to use pages again"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("page_size", [4, 12, 32, 64, 128])
@pytest.mark.parametrize("name,family", [("A", "mixed"), ("D", "mixed"), ("D", "last32"), ("E", "portions")])
def test_replay_at_other_page_sizes(models, tmp_path, name, family, page_size, dtype):
    """Pages of 4 to 128 tokens, among them a size that is no power of two: the matrix-core attention kernels take pages
    of 8 to 64 tokens, the others run the plain kernels; pages are still used again."""
    folder, cfg, requests, plain = models[name]
    steps = {"last32": tt.last_tokens_one_by_one, "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=6, refeed=[rid for rid, t in r.items() if len(t) >= 60][:1])}[family](requests)
    steps = tt.number(steps)
    runner = make_runner(folder, dtype, page_size, tt.live_tokens_bound(steps, round_to=max(64, page_size)))
    handed_out = tt.record_allocations(runner.cache)
    got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path))
    check(got, plain, dtype, f"{name} {dtype} {family} page {page_size}")
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools), "pages were lost"
    for pages in handed_out:
        assert len(pages) > len(set(pages)), "the trace was meant to use pages again"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_single_rows_beside_portions_take_the_decode_kernel(models, tmp_path, monkeypatch, name, dtype):
    """In a step that mixes portions of prompts with single tokens the single rows go to the decode kernel once their
    contexts are long; here from the first key on, so that the tiny models take that way."""
    from fllm_amd.parts.attention import PagedAttention
    monkeypatch.setattr(PagedAttention, "SPLIT_SINGLE_ROWS_FROM", 0)
    folder, cfg, requests, plain = models[name]
    steps = tt.number(tt.mixed(requests, seed=13, decode_tail=40))
    runner = make_runner(folder, dtype, tc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
    got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path))
    check(got, plain, dtype, f"{name} {dtype} mixed, single rows apart")
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    """bin/trace_run as a user starts it: steps on stdin, `done` lines back, files in --out."""
    folder, cfg, requests, plain = models["A"]
    steps = tt.number(tt.mixed(requests, seed=9))
    got = tt.run_subprocess(folder, dtype, steps, cfg["vocab_size"], str(tmp_path), tt.live_tokens_bound(steps))
    check(got, plain, dtype, f"trace_run {dtype}")


def test_cuts_agree_bit_for_bit_in_float32(models, tmp_path):
    """float32: every output element is one fixed chain of operations, so the way requests are
    cut into steps and batched changes nothing at all."""
    folder, cfg, requests, plain = models["B"]
    results = []
    for i, make in enumerate([tt.whole, tt.portions, lambda r: tt.mixed(r, seed=3)]):
        steps = tt.number(make(requests))
        runner = make_runner(folder, "float32", 8, tt.live_tokens_bound(steps))
        sub = tmp_path / str(i)
        results.append(tt.run_in_process(runner, steps, cfg["vocab_size"], str(sub)))
    for rid in requests:
        assert np.array_equal(results[0][rid], results[1][rid]), f"whole vs portions differ for {rid}"
        assert np.array_equal(results[0][rid], results[2][rid]), f"whole vs mixed differ for {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decoding(models, tmp_path, dtype):
    """A request decoded token by token from its very first token, up to the context limit."""
    folder, cfg, requests, plain = models["B"]
    rid = "r4"                                   # 256 tokens: the whole context of config B
    one = {rid: requests[rid]}
    steps = tt.number(tt.last_tokens_one_by_one(one, tail=256))
    runner = make_runner(folder, dtype, 8, 256)
    got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path))
    check(got, {rid: plain[rid]}, dtype, f"token by token {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_decode_graphs_and_eager_steps_agree(models, tmp_path, name, dtype):
    """Decode steps replay captured HIP graphs; every replay (with eager steps and synchronisations
    between them) gives what the eager step gives."""
    folder, cfg, requests, plain = models[name]
    steps = tt.number(tt.last_tokens_one_by_one(requests) + tt.mixed(requests, seed=21, decode_tail=40))
    results = []
    for i, use_graphs in enumerate((True, False)):
        runner = make_runner(folder, dtype, tc.PAGE_SIZES[name], tt.live_tokens_bound(steps), use_graphs=use_graphs)
        results.append(tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path / str(i))))
        assert (runner.graph_replays > 30) == use_graphs
    for rid, want in plain.items():
        a, b = results[0][rid].astype(np.float64), results[1][rid].astype(np.float64)
        if dtype == "float32":
            assert np.array_equal(a, b), f"{rid}: graph and eager steps differ in float32"
        else:
            assert np.abs(a - b).max() <= TOL[dtype] * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,count", [("A", 100), ("B", 75)])
def test_decode_steps_of_many_requests(models, tmp_path, name, count, dtype):
    """Decode steps of 65 to 128 requests are padded to 80, 96, 112 or 128 rows and replayed as graphs like the smaller
    ones: every request's logits are those of the plain implementation, and the rows that pad a step store nothing."""
    from fllm_amd.engine import ModelRunner
    folder, cfg, _, _ = models[name]
    from safetensors.torch import load_file
    w64 = tc.to_float64(load_file(os.path.join(folder, "model.safetensors")))
    lengths = [6 + (i * 7) % 5 for i in range(count)]              # 6 to 10 tokens: requests end at different steps
    requests = {f"n{i}": tc.random_ids(n, cfg["vocab_size"], 900 + i) for i, n in enumerate(lengths)}
    plain = {rid: plain_llama.forward(cfg, w64, toks) for rid, toks in requests.items()}
    head = 4
    steps = [{"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))} for rid, toks in requests.items()], "end": []}]
    for at in range(head, max(lengths)):
        live = {rid: toks for rid, toks in requests.items() if len(toks) > at}
        steps.append({"entries": [{"id": rid, "tokens": [toks[at]], "want": [0]} for rid, toks in live.items()],
                      "end": [rid for rid, toks in live.items() if len(toks) == at + 1]})
    runner = ModelRunner.from_folder(folder, dtype=dtype, page_size=tc.PAGE_SIZES[name], max_tokens=count * 64, max_requests=count)
    got = tt.run_in_process(runner, tt.number(steps), cfg["vocab_size"], str(tmp_path / "many"))
    check(got, plain, dtype, f"many {name} {dtype}")
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools)
    if runner.use_graphs:
        rows_seen = {key[0] for key in runner._graphs}
        assert rows_seen & {80, 96, 112, 128}, f"decode graphs of {sorted(rows_seen)} rows ran"
