"""Whole steps of the engine at the layer sizes that the benchmark times (Llama-3.1-8B, Llama-3.2-1B and
Llama-3.1-70B widths, with few layers and a small vocabulary), against the plain implementation: requests whole, in
portions, with the last tokens one by one, mixed with four live requests, and decoded in batches of 64, 40, 24, 8 and 1
rows through the captured graphs, in float32 and in bfloat16.  The kernel variants that only these sizes select (K
slices of the decode products, their 8-row tiles, eight query heads a key/value head, the tile-major copies of the
matrices and the fused forms of 17 to 48 rows that read them) run here inside a model; `options` is a model of such
widths with what the others lack: biases on every product, a sliding window on one layer, a partial rotary width.
The reference compares whole-model logits the same way (rust/engine/src/tiny_models.rs:946-1005,
scripts/verify_architectures.py:1-70)."""
import numpy as np
import pytest
import torch

import plain_llama
import tiny_configs as tc
import trace_tools as tt

pytestmark = pytest.mark.gpu

LLAMA3 = {"rope_type": "llama3", "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}


def config(layers, hidden, heads, kv_heads, head_dim, inter, factor, tied):
    return {"model_type": "llama", "architectures": ["LlamaForCausalLM"], "num_hidden_layers": layers, "hidden_size": hidden,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim, "intermediate_size": inter,
            "vocab_size": 1000, "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "rope_scaling": dict(LLAMA3, factor=factor),
            "tie_word_embeddings": tied, "max_position_embeddings": 1024, "hidden_act": "silu"}


SIZES = {
    "8b": config(2, 4096, 32, 8, 128, 14336, 8.0, False),
    "1b": config(2, 2048, 32, 8, 64, 8192, 32.0, True),
    "70b": config(1, 8192, 64, 8, 128, 28672, 8.0, False),
    "options": dict(config(2, 1024, 8, 2, 128, 3072, 8.0, True), partial_rotary_factor=0.5, sliding_window=40,
                    layer_types=["sliding_attention", "full_attention"]),
}
# |engine - plain| <= tol * max|plain logit|, and the engine's largest logit of every row is the plain implementation's
# or within twice that of it.  Largest errors seen on the MI355X: float32 9.1e-6; bfloat16 1.5e-2 (8b),
# 1.2e-2 (1b), 1.4e-2 (70b).  The plain kernels (one float32 chain per element, bfloat16 only where tensors are stored)
# are as far from the plain implementation at these widths (1.3e-2 at the 8b sizes): the distance is the storage type's.
TOL = {"float32": 2e-5, "bfloat16": 2e-2}
LADDER = [10] * 24 + [12] * 16 + [14] * 16 + [18] * 7 + [22]          # 64 requests; 64, 40, 24, 8 and 1 of them are left as they end


@pytest.fixture(scope="module")
def cases():
    """Per size: configuration, tensors (bfloat16-exact float32), requests and the plain logits; made at first use."""
    made = {}

    def get(name):
        if name not in made:
            from fllm_amd.registry import model_spec_from_config
            from fllm_amd.weights import random_tensors
            cfg = SIZES[name]
            _, spec = model_spec_from_config(cfg)
            tensors = {k: v.to(torch.float32) for k, v in random_tensors(spec, 77, torch.bfloat16, with_optional=(name == "options")).items()}
            lengths = {"w": 300, "m0": 90, "m1": 150, "m2": 60, "m3": 200}
            requests = {rid: tc.random_ids(n, cfg["vocab_size"], 7 + i) for i, (rid, n) in enumerate(lengths.items())}
            ladder = {f"d{i}": tc.random_ids(n, cfg["vocab_size"], 500 + i) for i, n in enumerate(LADDER)}
            w64 = tc.to_float64(tensors)
            plain = {rid: plain_llama.forward(cfg, w64, toks) for rid, toks in {**requests, **ladder}.items()}
            del w64
            made.clear()                      # one size at a time in memory
            made[name] = (cfg, spec, tensors, requests, ladder, plain)
        return made[name]

    return get


def ladder_steps(ladder, head=6):
    """The first `head` tokens of all requests in one step, then one token of every live request a step."""
    steps = [{"entries": [{"id": rid, "tokens": toks[:head], "want": list(range(head))} for rid, toks in ladder.items()],
              "end": []}]
    for at in range(head, max(len(t) for t in ladder.values())):
        live = {rid: toks for rid, toks in ladder.items() if len(toks) > at}
        steps.append({"entries": [{"id": rid, "tokens": [toks[at]], "want": [0]} for rid, toks in live.items()],
                      "end": [rid for rid, toks in live.items() if len(toks) == at + 1]})
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["8b", "1b", "70b", "options"])
def test_steps_at_benchmark_sizes(cases, tmp_path, name, dtype):
    from fllm_amd.engine import ModelRunner
    cfg, spec, tensors, requests, ladder, plain = cases(name)
    runner = ModelRunner(spec, tensors, dtype=dtype, page_size=16, max_tokens=64 * 64, max_requests=64)
    families = {
        "whole": tt.whole(requests),
        "last32": tt.last_tokens_one_by_one({"w": requests["w"]}),
        "portions": tt.portions({k: requests[k] for k in ("w", "m1")}),
        "mixed": tt.mixed(requests, seed=5),
        "batches": ladder_steps(ladder),
    }
    worst = {}
    for family, steps in families.items():
        steps = tt.number(steps)
        got = tt.run_in_process(runner, steps, cfg["vocab_size"], str(tmp_path / family))
        for rid, logits in got.items():
            want = plain[rid]
            assert logits.shape == want.shape, (family, rid)
            err = np.abs(logits.astype(np.float64) - want).max(axis=1) / np.abs(want).max()
            worst[family] = max(worst.get(family, 0.0), float(err.max()))
            tt.observe(f"benchmark sizes {name} {dtype}", err.max())
            assert err.max() <= TOL[dtype], (f"{name} {dtype} {family}: request {rid}: error {err.max():.3e} of the largest logit at "
                                             f"position {int(err.argmax())}; first position over the limit: "
                                             f"{int(np.argmax(err > TOL[dtype]))}")
            # the greedy token of every row: the plain implementation's, or one that nearly ties with it there
            chosen, best = logits.argmax(axis=1), want.argmax(axis=1)
            rows = np.arange(len(want))
            gap = (want[rows, best] - want[rows, chosen]) / np.abs(want).max(axis=1)
            assert gap.max() <= 2 * TOL[dtype], (f"{name} {dtype} {family}: request {rid}: position {int(gap.argmax())} takes token "
                                                 f"{int(chosen[gap.argmax()])}, the plain implementation {int(best[gap.argmax()])}")
        runner.cache.check_invariants()
        assert all(pool.available == pool.num_pages for pool in runner.cache.pools)
    print(f"observed errors {name} {dtype}: " + ", ".join(f"{k} {v:.2e}" for k, v in worst.items()))
    if dtype == "bfloat16":
        rows_seen = {key[0] for key in runner._graphs}
        assert {1, 8, 24, 40, 64} <= rows_seen, f"decode graphs of {sorted(rows_seen)} rows ran"
        ops = runner.rt.ops                      # the steps of 24 and 40 rows ran the fused forms that read the copies
        for block in runner.model.blocks:
            assert ops.fused_form(24, cfg["hidden_size"], block.mixer.w_qkv) == "chunks"
            assert ops.fused_form(40, cfg["hidden_size"], block.feed_forward.w_gate_up, gate_up=True) == "chunks"
            large = block.feed_forward.w_gate_up.numel() * 2 >= ops.OWN_GATE_UP_BYTES       # small matrices: the library's products
            assert ops.own_feed_forward(64, block.feed_forward.w_gate_up, block.feed_forward.w_down) == large
            # and so did the whole request of 90 tokens (six row tiles a workgroup), but no step of more than 128 rows
            assert ops.own_feed_forward(90, block.feed_forward.w_gate_up, block.feed_forward.w_down) == large
            assert not ops.own_feed_forward(150, block.feed_forward.w_gate_up, block.feed_forward.w_down)
