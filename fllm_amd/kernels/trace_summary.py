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


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(prog="fllm_amd trace-summary")
    ap.add_argument("path", help="a rocprofv3 output folder or a *kernel_trace.csv")
    ap.add_argument("--steps", type=int, default=8, help="engine steps to add up, counted back from the last one")
    ap.add_argument("--top", type=int, default=20)
    args = ap.parse_args(argv)
    print("\n".join(summarize(args.path, args.steps, args.top)))
    return 0
