#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X, Llama-3.1-8B sizes, random bfloat16
weights, synthetic token ids.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers N] [--shape 8b|1b|70b] [--no-further]

A step is one decode step of the whole engine (scheduler, step function, sampling), with steps
launched ahead of the tokens of the step before them (--no-ahead: each step waits for the last).  Every headline
figure (batch 1, 8, 64 and the prefill) is the median of --repeats (3) timed runs of K steps, each with requests of its own;
"runs_ms_per_step" lists them all.  "kernels" gives the device time of the kernels a batch-8 decode step and a prefill
step spend most on, in microseconds a step, from a short profiled run behind the timed ones.  The one
JSON line on standard output holds decoded tokens per second at the default batch (8), the same
at batch 1 and 64 under "points", a 2,048-token prefill under "prefill" and the decode step's
share of the HBM roofline under "roofline": of the published peaks (8 TB/s, 2.5 PFLOP/s), and under "measured_peak" /
"frac_measured" of what a kernel that only reads, or only issues MFMA products, gets out of this device.  Further points
(left out with --no-further): decoding at the default batch with sampled tokens (temperature 0.8, top-k 50, top-p 0.9) and at contexts of 8,192 and 32,768 tokens, and at the
Llama-3.2-1B sizes decoding one request and the mixed workload of 64 requests, each decode point with its share of
the roofline ("..._hbm_frac").
"""
import argparse
import json
import sys
import time

HBM_PEAK_GBS = 8000.0            # MI355X, published
MFMA_PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA_31_8B = {
    "model_type": "llama", "architectures": ["LlamaForCausalLM"],
    "num_hidden_layers": 32, "hidden_size": 4096, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
    "intermediate_size": 14336, "vocab_size": 128256, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
    "tie_word_embeddings": False, "max_position_embeddings": 131072, "hidden_act": "silu",
}
SHAPES = {
    "8b": LLAMA_31_8B,
    "1b": dict(LLAMA_31_8B, num_hidden_layers=16, hidden_size=2048, num_attention_heads=32, num_key_value_heads=8, head_dim=64,
               intermediate_size=8192, tie_word_embeddings=True,
               rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                             "original_max_position_embeddings": 8192}),
    "70b": dict(LLAMA_31_8B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=28672),
}
SHAPE_NAMES = {"8b": "Llama-3.1-8B shape", "1b": "Llama-3.2-1B shape", "70b": "Llama-3.1-70B shape"}
CONTEXT = 8192
PROMPT_LEN = 1024
PREFILL_TOKENS = 2048
PAGE_SIZE = 16
SAMPLED = {"temperature": 0.8, "top_k": 50, "top_p": 0.9}     # the sampled point of the default run


def linear_params(cfg, layers):
    h, nh, nkv, d, i = (cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"],
                        cfg["intermediate_size"])
    per_layer = h * (nh + 2 * nkv) * d + nh * d * h + 3 * h * i
    return per_layer * layers, cfg["vocab_size"] * h


def decode_step_bytes(cfg, layers, contexts, elem=2):
    """Bytes a decode step has to read: every weight it uses once, and the cache of the live requests."""
    body, head = linear_params(cfg, layers)
    norms = (2 * layers + 1) * cfg["hidden_size"] * 4
    kv = sum(contexts) * layers * 2 * cfg["num_key_value_heads"] * cfg["head_dim"] * elem
    return (body + head) * elem + norms + kv


def prefill_flops(cfg, layers, tokens):
    body, head = linear_params(cfg, layers)
    attention = layers * 4 * cfg["num_attention_heads"] * cfg["head_dim"] * (tokens * (tokens + 1) // 2)
    return 2 * tokens * body + 2 * head + attention          # the head runs on the one wanted row


def mixed_run(cfg, args, quiet=False):
    """Continuous batching under load: 64 requests at once, prompts of 64 to 2,048 tokens, 128 generated tokens each."""
    import numpy as np
    import torch
    from fllm_amd import Engine, SamplingParams
    rng = np.random.default_rng(1)
    lengths = rng.integers(64, 2049, 64).tolist()
    generate = 128
    need_tokens = sum(n + generate + PAGE_SIZE for n in lengths) + 64
    model = {k: v for k, v in cfg.items() if not k.startswith("_")}
    engine = Engine(config=model, seed=0, dtype="bfloat16", device="cuda:0", ctx=4096, max_seqs=64, max_batched_tokens=PREFILL_TOKENS,
                    block_size=PAGE_SIZE, num_blocks=-(-need_tokens // PAGE_SIZE), decode_first=True, random_weights_on_device=True,
                    ahead=not args.no_ahead)
    vocab = cfg["vocab_size"]
    results = []
    for run in range(2):            # the first run captures the graphs
        for i, n in enumerate(lengths):
            engine.add_request(f"m{run}-{i}", rng.integers(0, vocab, n).tolist(), SamplingParams(max_tokens=generate, ignore_eos=True))
        torch.cuda.synchronize()
        start, tokens, rounds = time.perf_counter(), 0, 0
        while engine.has_unfinished():
            tokens += len(engine.step())
            rounds += 1
        torch.cuda.synchronize()
        results.append((time.perf_counter() - start, tokens, rounds))
    elapsed, tokens, rounds = results[-1]
    assert tokens == 64 * generate
    record = {"workload": "64 requests at once, prompts of 64..2,048 tokens, 128 generated tokens each", "model": cfg.get("_name", ""),
              "seconds": round(elapsed, 3), "steps": rounds, "prompt_tokens": int(sum(lengths)),
              "generated_tokens": tokens, "generated_tokens_per_s": round(tokens / elapsed, 1),
              "all_tokens_per_s": round((tokens + sum(lengths)) / elapsed, 1), "preemptions": engine.stats.preemptions}
    if not quiet:
        print(json.dumps(record), flush=True)
    return record, engine


def decode_slack(batch, prompt_len):
    """Tokens a request may generate before the timed steps begin: a request whose prompt is done decodes while the
    prompts of the others still run, a step of PREFILL_TOKENS tokens at a time."""
    return batch * -(-prompt_len // PREFILL_TOKENS) + 8


def decode_run(engine, rng, vocab, batch, steps, warmup, prompt_len, tag, sampling=None):
    """`batch` requests with prompts of `prompt_len` tokens; the prompts run untimed, then `warmup` untimed and `steps`
    timed decode steps.  `sampling`: temperature, top_k, top_p of every request (greedy without).
    Returns (tokens/s, ms a step, mean context of each request over the timed steps)."""
    import torch
    from fllm_amd import SamplingParams
    params = SamplingParams(max_tokens=warmup + steps + decode_slack(batch, prompt_len), ignore_eos=True, **(sampling or {}))
    names = []
    for i in range(batch):
        name = f"{tag}-{i}"
        engine.add_request(name, rng.integers(0, vocab, prompt_len).tolist(), params)
        names.append(name)
    # prompts first (untimed): until every request has produced its first token
    produced = {n: 0 for n in names}
    while min(produced.values()) < 1:
        for ev in engine.step():
            produced[ev.request_id] += 1
    for _ in range(warmup - 1 if warmup > 0 else 0):
        engine.step()
    torch.cuda.synchronize()
    contexts = [engine.runner.cache.length(sid) for sid in engine.scheduler.running]
    start = time.perf_counter()
    tokens = 0
    for _ in range(steps):
        tokens += len(engine.step())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - start
    assert tokens == batch * steps, f"{tokens} tokens from {steps} steps of batch {batch}"
    for n in names:
        engine.abort_request(n)
    while engine.has_unfinished():          # the step that was launched ahead
        engine.step()
    return tokens / elapsed, elapsed / steps * 1e3, [c + steps / 2.0 for c in contexts]


def median_run(runs):
    """Of several (tokens/s, ms a step, contexts) the one with the median time a step."""
    ordered = sorted(runs, key=lambda r: r[1])
    return ordered[len(ordered) // 2]


def short_kernel_name(name):
    """`void (anonymous namespace)::kernel<1, 2>(Args, int)` -> `kernel<1, 2>`; a mangled name -> its function's name;
    a kernel of the GEMM library -> `gemm_library_MT<its tile>`."""
    import re
    tile = re.search(r"Cijk_.*?(MT\d+x\d+x\d+)", name)
    if tile:
        return "gemm_library_" + tile.group(1)
    mangled = re.match(r"_ZN?(?:12_GLOBAL__N_1)?(\d+)", name)
    if mangled:
        return name[mangled.end():mangled.end() + int(mangled.group(1))]
    name = name.replace("void ", "").replace("(anonymous namespace)::", "")
    depth = 0
    for i, ch in enumerate(name):
        depth += ch == "<"
        depth -= ch == ">"
        if ch == "(" and depth == 0:
            return name[:i]
    return name


def kernel_breakdown(run_steps, steps, top=8):
    """Device time by kernel over `steps` calls of `run_steps()` (one engine step each), in microseconds a step: the
    `top` longest by name and the rest as "other".  What the reference prints as its BatchStats per phase
    (rust/engine/src/runtime.rs:20-40) is per kernel here.  None when the profiler gives nothing."""
    import torch
    from torch.profiler import ProfilerActivity, profile
    try:
        with profile(activities=[ProfilerActivity.CUDA]) as prof:
            for _ in range(steps):
                run_steps()
            torch.cuda.synchronize()
        by_name = {}
        for e in prof.key_averages():
            if e.device_time_total > 0:
                name = short_kernel_name(e.key)
                by_name[name] = by_name.get(name, 0.0) + e.device_time_total / steps
        rows = list(by_name.items())
    except Exception as exc:                                   # a profiler that cannot attach must not cost the run its line
        print(f"[bench] no kernel breakdown: {exc}", file=sys.stderr, flush=True)
        return None
    rows.sort(key=lambda r: -r[1])
    out = {name: round(us, 1) for name, us in rows[:top]}
    if rows[top:]:
        out["other"] = round(sum(us for _, us in rows[top:]), 1)
    out["total"] = round(sum(us for _, us in rows), 1)
    return out or None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=248, help="timed decode steps (with the warm-up: 256 generated tokens a request)")
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--repeats", type=int, default=3, help="timed runs of each headline figure; the median is reported")
    ap.add_argument("--no-kernels", action="store_true", help="skip the profiled steps that give the per-kernel times")
    ap.add_argument("--shape", choices=sorted(SHAPES), default="8b",
                    help="layer sizes: Llama-3.1-8B (the default, the headline configuration), Llama-3.2-1B or Llama-3.1-70B")
    ap.add_argument("--layers", type=int, default=None,
                    help="fewer layers than the model has (both numbers are reported)")
    ap.add_argument("--mixed", action="store_true",
                    help="instead of the headline run: 64 requests with prompts of 64 to 2,048 tokens and 128 generated tokens each, "
                         "all submitted at once (continuous batching, prompts in portions beside decoding requests); prints a "
                         "line of its own")
    ap.add_argument("--no-ceilings", action="store_true",
                    help="do not measure what the device delivers to a kernel that only reads or only multiplies")
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64, the prefill and the further points")
    ap.add_argument("--no-further", action="store_true",
                    help="skip the points beyond the headline configuration: decoding at contexts of 8,192 and 32,768 tokens, and "
                         "the Llama-3.2-1B sizes (decoding at batch 1 and the mixed workload of 64 requests)")
    ap.add_argument("--no-ahead", action="store_true", help="every step waits for the tokens of the step before it")
    ap.add_argument("--no-weight-tiles", action="store_true",
                    help="without the tile-major copies of the output and down projection matrices that decode steps of up to 16 rows read")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run the 2,048-token prefill steps alone and print their time (for profiling); no JSON line")
    ap.add_argument("--prompt-tokens", type=int, default=PREFILL_TOKENS,
                    help="with --prefill-only: length of the prompt; longer ones run in portions of 2,048 tokens")
    ap.add_argument("--prompt-len", type=int, default=PROMPT_LEN, help="prompt length of the decode runs (for profiling other contexts)")
    ap.add_argument("--sampled", action="store_true",
                    help="for profiling the sampling kernels: the decode runs draw with temperature 0.8, top-k 50 and top-p 0.9 under a "
                         "repetition penalty of 1.1 and report 5 log-probabilities a token (the headline run is greedy)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this engine runs on a single MI355X, --gpus {args.gpus} is not supported")
        sys.exit(2)

    import numpy as np
    import torch
    from fllm_amd import Engine, SamplingParams

    shape = SHAPES[args.shape]
    if args.layers is None:
        args.layers = shape["num_hidden_layers"]
    cfg = dict(shape, num_hidden_layers=args.layers)
    steps, warmup = args.steps, args.warmup
    if args.mixed:
        mixed_run(dict(cfg, _name=SHAPE_NAMES[args.shape]), args)
        return
    further = not (args.no_points or args.no_further or args.prefill_only) and args.shape == "8b"
    long_contexts = (8192, 32768) if further else ()
    long_steps = 32
    batches = [args.batch] if args.no_points or args.prefill_only else sorted({1, args.batch, 32, 64})
    prompt_tokens = args.prompt_tokens if args.prefill_only else PREFILL_TOKENS
    runs = [(b, args.prompt_len, steps) for b in batches] + [(args.batch, c, long_steps) for c in long_contexts]
    held = [prompt + warmup + count + decode_slack(b, prompt) for b, prompt, count in runs]      # tokens a request comes to hold
    need_tokens = max(b * (h + PAGE_SIZE) for (b, _, _), h in zip(runs, held)) + prompt_tokens + 64
    most_context = max([CONTEXT, prompt_tokens + 64] + [h + 64 for h in held])
    t0 = time.time()
    engine = Engine(config=cfg, seed=0, dtype="bfloat16", device="cuda:0", ctx=most_context, max_seqs=max(batches),
                    max_batched_tokens=PREFILL_TOKENS, block_size=PAGE_SIZE, num_blocks=-(-need_tokens // PAGE_SIZE),
                    decode_first=True, random_weights_on_device=True, ahead=not args.no_ahead,
                    decode_weight_tiles=False if args.no_weight_tiles else "auto")
    print(f"[bench] engine ready in {time.time() - t0:.1f}s", file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    vocab = cfg["vocab_size"]

    def prefill_run(repeats=4):
        """Prompts of 2,048 tokens, one request each, one step each (a longer prompt: in portions of 2,048).  All
        requests wait in the queue before the clock starts and the first one runs untimed, so the timed steps follow one
        another as they do under load; a device that idled for milliseconds before a step runs its first
        kernels slower (5 ms of idling cost a 2,048-token step 1.7 ms here).  Returns the seconds a prompt took."""
        for i in range(repeats + 2):
            engine.add_request(f"prefill-{prefill_run.serial}-{i}", rng.integers(0, vocab, prompt_tokens).tolist(),
                               SamplingParams(max_tokens=1, ignore_eos=True))
        prefill_run.serial += 1
        finished = 0
        while finished < 1:
            finished += sum(1 for ev in engine.step() if ev.finished)
        torch.cuda.synchronize()          # what was launched so far (a step ahead, perhaps) has run: it is not timed
        rows_before = engine.stats.prefill_rows
        start = time.perf_counter()
        while finished < repeats + 2:
            finished += sum(1 for ev in engine.step() if ev.finished)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - start
        rows = engine.stats.prefill_rows - rows_before
        assert rows >= repeats * prompt_tokens
        return elapsed * prompt_tokens / rows

    prefill_run.serial = 0

    if args.prefill_only:
        best = prefill_run(max(2, steps))
        print(f"[bench] prefill {prompt_tokens} tokens: {best * 1e3:.2f} ms, {prompt_tokens / best:.0f} tokens/s",
              file=sys.stderr, flush=True)
        return

    def share(result, model=cfg, layers=args.layers):
        return decode_step_bytes(model, layers, result[2]) / (result[1] * 1e-3) / 1e9 / HBM_PEAK_GBS

    results, all_runs = {}, {}
    repeats = max(1, args.repeats)
    for batch in batches:
        runs = [decode_run(engine, rng, vocab, batch, steps, warmup, args.prompt_len, f"b{batch}r{r}",
                           sampling=dict(SAMPLED, repetition_penalty=1.1, logprobs=5) if args.sampled else None)
                for r in range(repeats)]
        results[batch] = median_run(runs)
        all_runs[batch] = [round(r[1], 4) for r in runs]
        print(f"[bench] decode batch {batch}: {results[batch][0]:.1f} tok/s, {results[batch][1]:.3f} ms/step (median of "
              f"{', '.join(f'{r[1]:.3f}' for r in runs)})", file=sys.stderr, flush=True)

    value, ms_per_step, contexts = results[args.batch]
    step_bytes = decode_step_bytes(cfg, args.layers, contexts)
    achieved = step_bytes / (ms_per_step * 1e-3) / 1e9
    line = {
        "metric": f"decode tok/s at batch {args.batch} ({SHAPE_NAMES[args.shape]}, {args.prompt_len:,}-token prompts); points: batch 1/32/64; prefill: 2,048 tokens",
        "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic token ids, random-init weights N(0, 0.02)",
        "config": {"model": SHAPE_NAMES[args.shape], "layers": args.layers, "layers_of_model": shape["num_hidden_layers"],
                   "hidden": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": cfg["num_key_value_heads"],
                   "head_dim": cfg["head_dim"], "intermediate": cfg["intermediate_size"], "vocab": vocab,
                   "global_batch": args.batch, "prompt_len": args.prompt_len, "seq_len": CONTEXT, "kv_block": PAGE_SIZE,
                   "kv_dtype": "bf16", "prefill_tokens": PREFILL_TOKENS, "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
        "timed_runs": repeats, "value_of_runs": "median",
        "runs_ms_per_step": {f"decode_b{b}": v for b, v in all_runs.items()},
    }
    if not args.no_points:
        line["points"] = {"decode_b1": round(results[1][0], 2), "decode_b64": round(results[64][0], 2),
                          "decode_b32": round(results[32][0], 2)}
        for b in (1, 32, 64):
            line["points"][f"decode_b{b}_hbm_frac"] = round(share(results[b]), 4)
        prefills = sorted(prefill_run() for _ in range(repeats))
        best = prefills[len(prefills) // 2]
        flops = prefill_flops(cfg, args.layers, PREFILL_TOKENS)
        line["prefill"] = {"value": round(PREFILL_TOKENS / best, 1), "tokens": PREFILL_TOKENS, "ms": round(best * 1e3, 3),
                           "frac": round(flops / best / (MFMA_PEAK_TFLOPS["bf16"] * 1e12), 4),
                           "achieved_tflops": round(flops / best / 1e12, 1), "peak_tflops": MFMA_PEAK_TFLOPS["bf16"]}
        line["runs_ms_per_step"]["prefill"] = [round(p * 1e3, 3) for p in prefills]
        print(f"[bench] prefill {PREFILL_TOKENS} tokens: {best * 1e3:.2f} ms (median of "
              f"{', '.join(f'{p * 1e3:.2f}' for p in prefills)})", file=sys.stderr, flush=True)
        if not args.no_kernels:
            line["kernels"] = {}
            prompts = iter(range(10 ** 6))

            def one_prompt():
                engine.add_request(f"profiled-{next(prompts)}", rng.integers(0, vocab, PREFILL_TOKENS).tolist(),
                                   SamplingParams(max_tokens=1, ignore_eos=True))
                while engine.has_unfinished():
                    engine.step()

            one_prompt()
            found = kernel_breakdown(one_prompt, 2)
            if found:
                line["kernels"]["prefill_us"] = found
            # a decode batch of its own for the profiled steps: prompts, a few steps untimed, then five profiled steps
            names = [f"profiled-b{args.batch}-{i}" for i in range(args.batch)]
            for name in names:
                engine.add_request(name, rng.integers(0, vocab, args.prompt_len).tolist(),
                                   SamplingParams(max_tokens=64, ignore_eos=True))
            got = {n: 0 for n in names}
            while min(got.values()) < 4:
                for ev in engine.step():
                    got[ev.request_id] += 1
            found = kernel_breakdown(engine.step, 5)
            if found:
                line["kernels"][f"decode_b{args.batch}_us"] = found
            for name in names:
                engine.abort_request(name)
            while engine.has_unfinished():
                engine.step()
            for phase, found in line["kernels"].items():
                print(f"[bench] kernels, {phase}: " + ", ".join(f"{k} {v}" for k, v in found.items()), file=sys.stderr, flush=True)
    if further:
        # the same batch with sampled tokens (temperature 0.8, top-k 50, top-p 0.9): what the sampler adds to a step
        result = decode_run(engine, rng, vocab, args.batch, min(steps, 64), 2, args.prompt_len, "sampled",
                            sampling=SAMPLED)
        line["points"][f"decode_b{args.batch}_sampled"] = round(result[0], 2)
        print(f"[bench] decode batch {args.batch}, temperature 0.8, top-k 50, top-p 0.9: {result[0]:.1f} tok/s, {result[1]:.3f} ms/step",
              file=sys.stderr, flush=True)
    for context in long_contexts:
        # the same batch further into its requests: the cache of the live requests outweighs the weights
        result = decode_run(engine, rng, vocab, args.batch, long_steps, 2, context, f"c{context}")
        line["points"][f"decode_b{args.batch}_ctx{context}"] = round(result[0], 2)
        line["points"][f"decode_b{args.batch}_ctx{context}_hbm_frac"] = round(share(result), 4)
        print(f"[bench] decode batch {args.batch} at context {context}: {result[0]:.1f} tok/s, {result[1]:.3f} ms/step",
              file=sys.stderr, flush=True)
    if not args.no_ceilings:
        # beside the published peaks: what a kernel that only reads, or only multiplies, gets out of this device
        measured = engine.runner.rt.ops.measured_ceilings()
        line["roofline"]["measured_peak"] = round(measured["hbm_read_gbs"], 1)
        line["roofline"]["frac_measured"] = round(achieved / measured["hbm_read_gbs"], 4)
        if "prefill" in line:
            line["prefill"]["measured_peak_tflops"] = round(measured["mfma_bf16_tflops"], 1)
            line["prefill"]["frac_measured"] = round(flops / best / (measured["mfma_bf16_tflops"] * 1e12), 4)
        print(f"[bench] measured ceilings: {measured['hbm_read_gbs']:.0f} GB/s read, {measured['mfma_bf16_tflops']:.0f} TFLOP/s bf16 MFMA",
              file=sys.stderr, flush=True)
    if further:
        # the Llama-3.2-1B sizes: decoding one request (the fixed cost of a kernel weighs most there), and continuous
        # batching under load (64 requests at once, prompts of 64 to 2,048 tokens, 128 generated tokens each)
        del engine
        import gc
        gc.collect()
        torch.cuda.empty_cache()
        small = dict(SHAPES["1b"], _name=SHAPE_NAMES["1b"])
        record, small_engine = mixed_run(small, args, quiet=True)
        line["points"]["mixed_1b_generated_tok_s"] = record["generated_tokens_per_s"]
        line["points"]["mixed_1b_all_tok_s"] = record["all_tokens_per_s"]
        print(f"[bench] 1B sizes, 64 mixed requests: {record['generated_tokens_per_s']:.0f} generated tok/s, "
              f"{record['all_tokens_per_s']:.0f} tok/s with the prompts", file=sys.stderr, flush=True)
        model = {k: v for k, v in small.items() if not k.startswith("_")}
        result = decode_run(small_engine, rng, vocab, 1, steps, warmup, PROMPT_LEN, "s1")
        line["points"]["decode_1b_b1"] = round(result[0], 2)
        line["points"]["decode_1b_b1_hbm_frac"] = round(share(result, model, model["num_hidden_layers"]), 4)
        print(f"[bench] 1B sizes, decode batch 1: {result[0]:.1f} tok/s, {result[1]:.3f} ms/step", file=sys.stderr, flush=True)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
