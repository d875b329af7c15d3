"""The benchmark's line as the round's records read it: one JSON object with the agreed keys, the configuration flat,
both layer counts when fewer layers run, and a refusal of more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*flags, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True, timeout=timeout,
                          cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_one_line():
    done = run_bench("--gpus", "2", timeout=60)
    assert done.returncode == 2
    assert len(done.stdout.strip().splitlines()) == 1 and "one GPU" in done.stdout


@pytest.mark.gpu
def test_the_line_of_a_short_run():
    done = run_bench("--layers", "2", "--steps", "6", "--warmup", "2", "--no-further", "--no-ceilings")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = done.stdout.strip().splitlines()
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "prefill", "roofline", "points"):
        assert key in line, key
    assert (line["n_gpus"], line["steps"], line["warmup"], line["dtype"], line["unit"]) == (1, 6, 2, "bf16", "tokens/s")
    assert line["higher_is_better"] is True and line["value"] > 0
    assert abs(line["value"] - 8 / (line["ms_per_step"] * 1e-3)) < 0.01 * line["value"]        # 8 tokens a step
    config = line["config"]
    assert len(config) <= 20 and all(not isinstance(v, (dict, list)) for v in config.values())
    assert (config["layers"], config["layers_of_model"], config["global_batch"], config["hidden"]) == (2, 32, 8, 4096)
    assert set(line["prefill"]) >= {"value", "tokens", "ms", "frac"} and line["prefill"]["tokens"] == 2048
    assert abs(line["prefill"]["value"] - 2048 / (line["prefill"]["ms"] * 1e-3)) < 0.01 * line["prefill"]["value"]
    roofline = line["roofline"]
    assert (roofline["bound"], roofline["peak"], roofline["unit"]) == ("hbm", 8000.0, "GB/s")
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-3 and 0 < roofline["frac"] < 1
    assert line["points"]["decode_b1"] > 0 and line["points"]["decode_b64"] > line["points"]["decode_b1"]
    # every headline figure is the median of three timed runs, all of them listed
    runs = line["runs_ms_per_step"]
    assert line["timed_runs"] == 3 and set(runs) == {"decode_b1", "decode_b8", "decode_b32", "decode_b64", "prefill"}
    assert all(len(v) == 3 for v in runs.values())
    assert sorted(runs["decode_b8"])[1] == line["ms_per_step"] and sorted(runs["prefill"])[1] == line["prefill"]["ms"]
    flops = line["prefill"]["achieved_tflops"] * 1e12
    assert abs(flops / (line["prefill"]["peak_tflops"] * 1e12) - line["prefill"]["frac"]) < 1e-3
    # the kernels a step's time goes to, in microseconds a step: they add up to most of the step
    for phase, ms in (("decode_b8_us", line["ms_per_step"]), ("prefill_us", line["prefill"]["ms"])):
        kernels = line["kernels"][phase]
        assert len(kernels) >= 4 and 0.5 * ms * 1e3 < kernels["total"] < 1.2 * ms * 1e3, (phase, kernels, ms)
        assert abs(sum(v for k, v in kernels.items() if k != "total") - kernels["total"]) < 1.0


@pytest.mark.gpu
def test_the_smoke_run_of_the_entry_file():
    """`__graft_entry__.smoke()` in a process of its own, as it is run: a few tokens of a tiny random model on the
    device against the plain implementation."""
    done = subprocess.run([sys.executable, "-c", "import __graft_entry__ as g; g.smoke()"], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)
    assert done.returncode == 0, (done.stdout + done.stderr)[-2000:]
