"""Per-kernel time of the last engine steps in a `rocprofv3 --kernel-trace --output-format csv` run.

A whole run mixes the prompts' steps with the decode steps; every step of the engine begins with the
embedding kernel, so the trace is cut there and only the last steps are added up."""
from __future__ import annotations

import collections
import csv
import glob
import os
from typing import List


def find_trace(path: str) -> str:
    if os.path.isfile(path):
        return path
    found = sorted(glob.glob(os.path.join(path, "**", "*kernel_trace.csv"), recursive=True))
    if not found:
        raise FileNotFoundError(f"no *kernel_trace.csv under {path}")
    return found[-1]


def summarize(path: str, steps: int = 8, top: int = 20, marker: str = "embed_kernel") -> List[str]:
    with open(find_trace(path), newline="") as f:
        rows = list(csv.DictReader(f))
    rows.sort(key=lambda r: int(r["Start_Timestamp"]))
    starts = [i for i, r in enumerate(rows) if marker in r["Kernel_Name"]]
    if len(starts) < steps + 1:
        raise ValueError(f"the trace holds {len(starts)} steps, {steps + 1} are needed")
    # from the start of the step `steps` before the last one to the start of the last one
    sel = rows[starts[-steps - 1]: starts[-1]]
    total = collections.defaultdict(float)
    calls = collections.Counter()
    for r in sel:
        name = r["Kernel_Name"]
        total[name] += (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3
        calls[name] += 1
    span = (int(rows[starts[-1]]["Start_Timestamp"]) - int(sel[0]["Start_Timestamp"])) / 1e3
    busy = sum(total.values())
    lines = [f"{steps} steps: {span / steps:.1f} us a step from start to start, {busy / steps:.1f} us of it in kernels",
             f"{'us/step':>9} {'calls/step':>10} {'avg us':>8} {'share':>6}  kernel"]
    for name, t in sorted(total.items(), key=lambda kv: -kv[1])[:top]:
        lines.append(f"{t / steps:9.1f} {calls[name] / steps:10.1f} {t / calls[name]:8.2f} {t / busy:6.1%}  {name[:110]}")
    return lines


def find_counters(path: str) -> str:
    if os.path.isfile(path):
        return path
    found = sorted(glob.glob(os.path.join(path, "**", "*counter_collection.csv"), recursive=True))
    if not found:
        raise FileNotFoundError(f"no *counter_collection.csv under {path}")
    return found[-1]


def summarize_counters(path: str, last: int = 2000, top: int = 8) -> List[str]:
    """Hardware counters of a `rocprofv3 --pmc ... --output-format csv` run, averaged per dispatch for each kernel over
    the last `last` dispatches of the run (the decode steps at its end).  One row a kernel, one column a counter."""
    with open(find_counters(path), newline="") as f:
        rows = list(csv.DictReader(f))
    ids = sorted({int(r["Dispatch_Id"]) for r in rows})
    keep = set(ids[-last:])
    sums = collections.defaultdict(lambda: collections.defaultdict(float))
    dispatches = collections.defaultdict(set)
    names = []
    for r in rows:
        if int(r["Dispatch_Id"]) not in keep:
            continue
        kernel, counter = r["Kernel_Name"], r["Counter_Name"]
        if counter not in names:
            names.append(counter)
        sums[kernel][counter] += float(r["Counter_Value"])
        dispatches[kernel].add(int(r["Dispatch_Id"]))
    order = sorted(sums, key=lambda k: -len(dispatches[k]))[:top]
    lines = [f"counters a dispatch, averaged over the last {len(keep)} dispatches of the run"]
    for kernel in order:
        n = len(dispatches[kernel])
        lines.append(f"{kernel[:100]}  ({n} dispatches)")
        for counter in names:
            lines.append(f"    {counter:32s} {sums[kernel][counter] / n:16.1f}")
    return lines


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="fllm_amd trace-summary")
    ap.add_argument("path", help="a rocprofv3 output folder or a *kernel_trace.csv")
    ap.add_argument("--steps", type=int, default=8, help="engine steps to add up, counted back from the last one")
    ap.add_argument("--top", type=int, default=20)
    ap.add_argument("--counters", action="store_true",
                    help="the folder holds a --pmc run: print the counters a dispatch for each kernel instead")
    ap.add_argument("--last", type=int, default=2000, help="with --counters: dispatches to average over, counted back from the end")
    args = ap.parse_args(argv)
    if args.counters:
        print("\n".join(summarize_counters(args.path, args.last, min(args.top, 8))))
    else:
        print("\n".join(summarize(args.path, args.steps, args.top)))
    return 0
