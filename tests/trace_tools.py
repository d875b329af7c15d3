"""Traces for the replay tests: the same requests cut into steps in different ways."""
import json
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PORTIONS = [7, 2, 13, 3, 32, 2, 11, 5, 64, 2]


# Largest |engine - plain| / max |plain logit| that each group of comparisons saw in this run; the test session prints
# them at its end (tests/conftest.py), which is where the tolerances of the bfloat16 comparisons come from.
OBSERVED = {}


def observe(group, value):
    OBSERVED[group] = max(OBSERVED.get(group, 0.0), float(value))


def whole(requests):
    """Each request alone, in one step, logits wanted everywhere."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]})
    return steps


def last_tokens_one_by_one(requests, tail=32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(0, len(toks) - tail)
        if head:
            steps.append({"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))}], "end": []})
        for i in range(head, len(toks)):
            steps.append({"entries": [{"id": rid, "tokens": [toks[i]], "want": [0]}], "end": []})
        steps[-1]["end"] = [rid]
    return steps


def portions(requests, sizes=PORTIONS):
    """Portions of changing size, down to two tokens."""
    steps = []
    turn = 0
    for rid, toks in requests.items():
        i = 0
        while i < len(toks):
            n = min(sizes[turn % len(sizes)], len(toks) - i)
            turn += 1
            steps.append({"entries": [{"id": rid, "tokens": toks[i:i + n], "want": list(range(n))}], "end": []})
            i += n
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests, seed, max_live=4, decode_tail=12, refeed=()):
    """Up to `max_live` requests at a time: portions of some beside single tokens of others;
    a request sometimes sits a step out; finished requests leave and the next one arrives.
    A request named in `refeed` is ended once it has been fed about half of its tokens (what it holds is given
    back) and is fed again from its first token under the same name while the others go on, as a scheduler does
    that preempts a request and computes it again."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live = {}      # id -> (tokens, fed)
    again = set(refeed)
    steps = []
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0]
        entries, ends = [], []
        for rid in list(live):
            toks, fed = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                         # left out of this step
            rest = len(toks) - fed
            if rest <= decode_tail:
                n = 1                                            # "decoding": one token a step
            else:
                n = int(min(rest - decode_tail, rng.choice([2, 3, 5, 8, 16, 27, 40])))
            entries.append({"id": rid, "tokens": toks[fed:fed + n], "want": list(range(n))})
            live[rid][1] = fed + n
            if fed + n == len(toks):
                ends.append(rid)
                del live[rid]
            elif rid in again and fed + n >= len(toks) // 2:
                again.discard(rid)
                ends.append(rid)                                 # given up half way ...
                del live[rid]
                waiting.insert(0, (rid, toks))                   # ... and next in line, from its first token
        if entries:
            steps.append({"entries": entries, "end": ends})
    return steps


def number(steps, first=0):
    return [dict(step=first + i, **s) for i, s in enumerate(steps)]


def live_tokens_bound(steps, round_to=64):
    """Most tokens live requests hold at any time, each rounded up to `round_to`."""
    held, most = {}, 0
    for s in steps:
        for e in s["entries"]:
            held[e["id"]] = held.get(e["id"], 0) + len(e["tokens"])
        most = max(most, sum(-(-n // round_to) * round_to for n in held.values()))
        for rid in s["end"]:
            held.pop(rid, None)
    return most


def collect(steps, read_step, vocab, given_up=None):
    """Per request the logits of every position, in position order: id -> [tokens, vocab].  Of a request that was
    ended and fed again this is the last feeding; what the feedings before it gave goes to `given_up`
    (id -> list of [tokens fed, vocab]) when that is a dict."""
    out = {}
    ended = set()
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        data = read_step(s["step"]).reshape(wanted, vocab) if wanted else None
        o = 0
        for e in s["entries"]:
            n = len(e["want"])
            assert e["want"] == list(range(len(e["tokens"]))), "these traces want every position"
            if e["id"] in ended:                                  # fed again from its first token
                ended.discard(e["id"])
                if given_up is not None:
                    given_up.setdefault(e["id"], []).append(np.concatenate(out[e["id"]]))
                out[e["id"]] = []
            out.setdefault(e["id"], []).append(data[o:o + n])
            o += n
        ended.update(s["end"])
    return {k: np.concatenate(v) for k, v in out.items()}


def run_in_process(runner, steps, vocab, out_dir, given_up=None):
    import io
    from fllm_amd.engine.replay import replay
    log = io.StringIO()
    replay(runner, [json.dumps(s) for s in steps], out_dir, out=log)
    assert log.getvalue().split() == [w for s in steps for w in ("done", str(s["step"]))]
    return collect(steps, lambda i: np.fromfile(os.path.join(out_dir, f"{i}.f32"), dtype="<f4"), vocab, given_up)


def run_subprocess(model_dir, dtype, steps, vocab, out_dir, max_tokens, env=None):
    """Drives bin/trace_run the way a user does: a step goes in only after `done` came back."""
    cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, env=env)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline()
            assert line.strip() == f"done {s['step']}", f"expected 'done {s['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    return collect(steps, lambda i: np.fromfile(os.path.join(out_dir, f"{i}.f32"), dtype="<f4"), vocab)


def record_allocations(cache):
    """Per cache group the pages the pool hands out from now on, in order."""
    handed_out = [[] for _ in cache.pools]

    def wrap(pool, log):
        original = pool.alloc

        def alloc():
            page = original()
            log.append(page)
            return page
        pool.alloc = alloc

    for pool, log in zip(cache.pools, handed_out):
        wrap(pool, log)
    return handed_out
