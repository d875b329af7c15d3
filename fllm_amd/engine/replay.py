"""Trace replay: feeds given token ids through the engine's own step function, step by step, and
writes the logits at the wanted places.  It samples nothing and has no forward pass, cache or
loader of its own.  (The reference's nearest tool is rust/engine/examples/verify_checkpoint.rs:1-58.)

Input, one JSON object per line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
Output: `<out>/<step>.f32` (little-endian float32 [wanted, vocab]) for steps that want something,
and a line `done <step>` on standard output after every step.
"""
from __future__ import annotations

import json
import os
import sys
from typing import IO

from .runner import ModelRunner, StepEntry


def replay(runner: ModelRunner, lines: IO[str], out_dir: str, out: IO[str] = sys.stdout) -> int:
    os.makedirs(out_dir, exist_ok=True)
    steps = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = [StepEntry(e["id"], e["tokens"], e.get("want", [])) for e in record.get("entries", [])]
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                data = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                data.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for req_id in record.get("end", []):
            runner.free_request(req_id)
        out.write(f"done {step}\n")
        out.flush()
        steps += 1
    return steps


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--device", default="cuda:0")
    args = ap.parse_args(argv)
    if 64 % args.page_size != 0:
        ap.error("--page-size must divide 64")
    print("[trace_run] loading kernels and model ...", file=sys.stderr, flush=True)
    runner = ModelRunner.from_folder(args.model, dtype=args.dtype, device=args.device, page_size=args.page_size,
                                     max_tokens=args.max_tokens, max_requests=8)
    print("[trace_run] ready", file=sys.stderr, flush=True)
    replay(runner, sys.stdin, args.out)
    return 0
