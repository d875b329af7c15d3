"""Command line: `python -m fllm_amd <command>`.

Commands and option names follow the reference's binary where it has them
(rust/engine/src/cli.rs:16-170 dispatch; rust/engine/src/bin/serve.rs:530-557, :589-613, :681-782
flags; rust/engine/src/tiny_model.rs:168-195 `make-tiny-model`; rust/engine/src/backend/selftest.rs:48-71
`selftest-gpu`).  Text in and out is token ids: there is no tokenizer here.

    run MODEL --prompt-ids 1,2,3 [--prompt-ids ...] | --prompts-file FILE   generate
    inspect MODEL                                                          configuration and tensor check
    make-tiny-model OUT [--seed N] [--config FILE] [--dtype float32|bfloat16]
    selftest-gpu [--only GROUPS] [--list]                                   kernels against PyTorch on the device
    replay --model DIR --dtype D --out DIR --max-tokens N                   same as bin/trace_run
    trace-summary DIR [--steps N | --counters [--last N]]                   per-kernel time of the last steps of a rocprofv3 trace, or counters a dispatch of a --pmc run
"""
from __future__ import annotations

import argparse
import json
import sys
import time
from typing import List


def _engine_options(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--ctx", "--max-model-len", dest="ctx", type=int, default=None, help="context per sequence")
    ap.add_argument("--max-seqs", type=int, default=16, help="concurrent sequences")
    ap.add_argument("--max-batched-tokens", type=int, default=512, help="token budget of a step")
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--kv-block-size", type=int, default=16)
    ap.add_argument("--kv-blocks", type=int, default=None, help="cache pages (default: what fits)")
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.90)
    ap.add_argument("--kv-watermark-blocks", type=int, default=0)
    ap.add_argument("--max-num-partial-prefills", type=int, default=0)
    ap.add_argument("--long-prefill-token-threshold", type=int, default=0)
    ap.add_argument("--max-long-partial-prefills", type=int, default=1,
                    help="prompts longer than the threshold that may be in their portions at once")
    ap.add_argument("--preemption-mode", default="recompute", choices=["recompute", "none"])
    ap.add_argument("--scheduling-policy", default="fcfs", choices=["fcfs", "priority"])
    ap.add_argument("--prefix-cache", action="store_true", default=None,
                    help="keep full cache pages after their request and start later requests behind the tokens they share "
                         "(default: the environment's FLLM_PREFIX_CACHE, else off)")
    ap.add_argument("--chunked-prefill-policy", default="decode-first", choices=["decode-first", "prefill-first"])
    ap.add_argument("--no-ahead", dest="ahead", action="store_false",
                    help="wait for the tokens of every step before the next one is launched (by default a step is launched "
                         "while the tokens of the step before it are still on their way to the host)")
    ap.add_argument("--warm-up", action="store_true",
                    help="before the first request: capture the decode graphs of every batch size and run the sampler and prompt portions once")
    ap.add_argument("--check-layers", type=int, default=0, metavar="STEPS",
                    help="run every layer of the first STEPS steps also with the plain kernels and print their distance layer by layer")


def _make_engine(args, model):
    from . import Engine
    return Engine(model, dtype=args.dtype, device=args.device, ctx=args.ctx, max_seqs=args.max_seqs,
                  max_batched_tokens=args.max_batched_tokens, block_size=args.kv_block_size, num_blocks=args.kv_blocks,
                  gpu_memory_utilization=args.gpu_memory_utilization, kv_watermark_blocks=args.kv_watermark_blocks,
                  max_num_partial_prefills=args.max_num_partial_prefills,
                  long_prefill_token_threshold=args.long_prefill_token_threshold,
                  max_long_partial_prefills=args.max_long_partial_prefills, preemption_mode=args.preemption_mode,
                  decode_first=args.chunked_prefill_policy == "decode-first", ahead=args.ahead,
                  scheduling_policy=args.scheduling_policy, prefix_cache=args.prefix_cache,
                  check_layers=args.check_layers)


def cmd_run(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="fllm_amd run")
    ap.add_argument("model")
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids (repeatable)")
    ap.add_argument("--prompts-file", help="JSON file: a list of token id lists")
    ap.add_argument("--max-tokens", "--max-new", dest="max_tokens", type=int, default=64)
    ap.add_argument("--temperature", "--temp", dest="temperature", type=float, default=None, help="0: greedy (the default)")
    ap.add_argument("--top-p", type=float, default=None)
    ap.add_argument("--top-k", type=int, default=None)
    ap.add_argument("--generation-config", default="auto", metavar="auto|vllm|PATH",
                    help="where sampling defaults come from when a flag is left out: the model folder's generation_config.json "
                         "(auto), nowhere (vllm), or a file or folder named here; of its keys temperature, top_p, top_k, min_p "
                         "and repetition_penalty count")
    ap.add_argument("--no-generation-config", dest="generation_config", action="store_const", const="vllm",
                    help="the same as --generation-config vllm")
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--n", type=int, default=1, help="answers to every prompt (at most 16), each with draws of its own")
    ap.add_argument("--min-p", type=float, default=None, help="drop what weighs less than this share of the likeliest token")
    ap.add_argument("--repeat-penalty", type=float, default=None, help="repetition penalty on tokens seen before (1: off)")
    ap.add_argument("--presence-penalty", type=float, default=0.0)
    ap.add_argument("--frequency-penalty", type=float, default=0.0)
    ap.add_argument("--repeat-last-n", type=int, default=-1, help="tokens of the history the penalties look at (negative: all)")
    ap.add_argument("--min-tokens", type=int, default=0, help="no end-of-sequence or stop id before this many generated tokens")
    ap.add_argument("--logit-bias", default="", help="comma-separated id:value pairs added to the logits")
    ap.add_argument("--logprobs", type=int, default=None, metavar="N",
                    help="with every token its log-probability in the model's distribution and the N likeliest tokens (at most 20)")
    ap.add_argument("--logprobs-mode", choices=["raw_logprobs", "processed_logprobs"], default="raw_logprobs",
                    help="processed_logprobs: the log-probabilities are those of the distribution a token was drawn from "
                         "(after penalties, temperature and filters) instead of the model's own")
    ap.add_argument("--allowed-token-ids", default="", help="comma-separated: only these tokens can be chosen")
    ap.add_argument("--bad-words-ids", action="append", default=[], metavar="IDS",
                    help="comma-separated token ids of a sequence that must not be generated (repeatable)")
    ap.add_argument("--timeout", type=float, default=None, metavar="SECONDS", help="give a request up after this long")
    ap.add_argument("--stop-token-ids", default="", help="comma-separated")
    ap.add_argument("--ignore-eos", action="store_true")
    _engine_options(ap)
    args = ap.parse_args(argv)
    from . import SamplingParams
    from .config.files import generation_defaults
    import os
    defaults, origin = generation_defaults(args.generation_config, args.model if os.path.isdir(args.model) else None)
    if defaults:
        print(f"sampling defaults from {origin}: " + ", ".join(f"{k}={v}" for k, v in defaults.items()), file=sys.stderr)
    builtin = {"temperature": 0.0, "top_p": 1.0, "top_k": 0, "min_p": 0.0, "repetition_penalty": 1.0}
    given = {"temperature": args.temperature, "top_p": args.top_p, "top_k": args.top_k, "min_p": args.min_p,
             "repetition_penalty": args.repeat_penalty}
    chosen = {k: given[k] if given[k] is not None else defaults.get(k, builtin[k]) for k in builtin}
    prompts = [[int(t) for t in p.split(",") if t.strip()] for p in args.prompt_ids]
    if args.prompts_file:
        with open(args.prompts_file) as fh:
            prompts += json.load(fh)
    if not prompts:
        ap.error("give --prompt-ids or --prompts-file")
    engine = _make_engine(args, args.model)
    if args.warm_up:
        started = time.perf_counter()
        count = engine.warm_up()
        print(f"warm-up: {count} requests, {len(engine.runner._graphs)} decode graphs in {time.perf_counter() - started:.2f}s",
              file=sys.stderr)
    stops = tuple(int(t) for t in args.stop_token_ids.split(",") if t.strip())
    bias = tuple((int(t), float(b)) for t, b in (pair.split(":") for pair in args.logit_bias.split(",") if pair.strip()))
    params = SamplingParams(seed=args.seed, max_tokens=args.max_tokens, stop_token_ids=stops, ignore_eos=args.ignore_eos,
                            **chosen, presence_penalty=args.presence_penalty,
                            frequency_penalty=args.frequency_penalty, repeat_last_n=args.repeat_last_n,
                            min_tokens=args.min_tokens, logit_bias=bias, logprobs=args.logprobs,
                            logprobs_processed=args.logprobs_mode == "processed_logprobs",
                            allowed_token_ids=tuple(int(t) for t in args.allowed_token_ids.split(",") if t.strip()),
                            bad_word_ids=tuple(tuple(int(t) for t in w.split(",") if t.strip()) for w in args.bad_words_ids),
                            timeout_secs=args.timeout, n=args.n)
    names = [f"prompt-{i}" for i in range(len(prompts))]
    for name, prompt in zip(names, prompts):
        engine.add_request(name, prompt, params)
    outputs = {(n, k): [] for n in names for k in range(args.n)}
    logprobs = {(n, k): [] for n in names for k in range(args.n)}
    reasons = {}
    start = time.perf_counter()
    while engine.has_unfinished():
        for ev in engine.step():
            if ev.token_id >= 0:
                outputs[ev.request_id, ev.choice].append(ev.token_id)
            if ev.logprob is not None:
                logprobs[ev.request_id, ev.choice].append({"logprob": ev.logprob, "top": [[t, v] for t, v in ev.top_logprobs]})
            if ev.finished:
                for k in ([ev.choice] if ev.token_id >= 0 else range(args.n)):      # a timeout ends every answer
                    reasons.setdefault((ev.request_id, k), ev.finish_reason)
    elapsed = time.perf_counter() - start
    for name, prompt in zip(names, prompts):
        for k in range(args.n):
            record = {"request": name, "prompt_tokens": len(prompt), "token_ids": outputs[name, k], "finish_reason": reasons.get((name, k))}
            if args.n > 1:
                record["choice"] = k
            if args.logprobs is not None:
                record["logprobs"] = logprobs[name, k]
            print(json.dumps(record))
    st = engine.stats
    total = sum(len(v) for v in outputs.values())
    print(f"stats: forward_calls={st.forward_calls} rows_total={st.rows_total} max_rows={st.max_rows} "
          f"prefill_rows={st.prefill_rows} decode_rows={st.decode_rows} preemptions={st.preemptions} prefix_hit_tokens={st.prefix_hit_tokens} "
          f"scheduler={st.scheduler_s * 1e3:.1f}ms model_forward={st.forward_s * 1e3:.1f}ms "
          f"postprocess={st.postprocess_s * 1e3:.1f}ms; generated {total} tok in {elapsed:.3f}s "
          f"({total / max(elapsed, 1e-9):.1f} tok/s)", file=sys.stderr)
    return 0


def cmd_inspect(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="fllm_amd inspect")
    ap.add_argument("model")
    args = ap.parse_args(argv)
    from .config.files import read_config_json
    from .registry import model_spec_from_config
    from .weights.loader import canonical_names, check_tensors, expected_tensors
    from .weights.safetensors_io import open_checkpoint
    typed, spec = model_spec_from_config(read_config_json(args.model))
    print(f"architecture: {spec.architecture}")
    print(f"config: {typed}")
    required, _, _ = expected_tensors(spec)
    print(f"tensors expected: {len(required)}, parameters: {sum(int(__import__('math').prod(s)) for s in required.values()):,}")
    found = open_checkpoint(args.model)
    check_tensors(spec, {canonical: found[n][0].entries[n].shape for n, canonical in canonical_names(spec, found).items()})
    dtypes = sorted({f.entries[n].dtype for n, (f, _) in found.items()})
    print(f"checkpoint: {len(found)} tensors, stored as {', '.join(dtypes)}: ok")
    return 0


def cmd_make_tiny_model(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="fllm_amd make-tiny-model")
    ap.add_argument("out")
    ap.add_argument("--seed", type=int, default=0x0005EED0FF11)
    ap.add_argument("--config", help="config.json to take the sizes from (default: a two-layer Llama of width 64)")
    ap.add_argument("--dtype", default="float32", choices=["float32", "bfloat16"])
    args = ap.parse_args(argv)
    from .weights.random_init import write_random_model
    if args.config:
        with open(args.config) as fh:
            config = json.load(fh)
    else:
        # the sizes of the reference's tiny model (rust/engine/src/tiny_model.rs:11-17, :77-84)
        config = {"model_type": "llama", "architectures": ["LlamaForCausalLM"], "hidden_size": 64,
                  "num_attention_heads": 4, "num_key_value_heads": 2, "num_hidden_layers": 2, "intermediate_size": 128,
                  "vocab_size": 99, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "max_position_embeddings": 512,
                  "hidden_act": "silu", "tie_word_embeddings": False, "bos_token_id": 1, "eos_token_id": 2}
    write_random_model(args.out, config, args.seed, args.dtype)
    print(f"wrote {args.out}")
    return 0


def cmd_selftest(argv: List[str]) -> int:
    ap = argparse.ArgumentParser(prog="fllm_amd selftest-gpu")
    ap.add_argument("--only", default="", help="comma-separated groups")
    ap.add_argument("--list", action="store_true")
    args = ap.parse_args(argv)
    from .kernels import selftest
    if args.list:
        print("\n".join(selftest.GROUPS))
        return 0
    only = [g for g in args.only.split(",") if g]
    return selftest.run(only or None)


def cmd_replay(argv: List[str]) -> int:
    from .engine.replay import main
    return main(argv)


def cmd_trace_summary(argv: List[str]) -> int:
    from .kernels.trace_summary import main
    return main(argv)


COMMANDS = {"trace-summary": cmd_trace_summary, "run": cmd_run, "inspect": cmd_inspect, "make-tiny-model": cmd_make_tiny_model,
            "selftest-gpu": cmd_selftest, "replay": cmd_replay}


def main(argv=None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if not argv or argv[0] in ("-h", "--help"):
        print(__doc__)
        return 0
    cmd = COMMANDS.get(argv[0])
    if cmd is None:
        print(f"unknown command {argv[0]!r}; commands: {', '.join(COMMANDS)}", file=sys.stderr)
        return 2
    return cmd(argv[1:])
