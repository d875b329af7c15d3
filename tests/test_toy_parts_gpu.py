"""A toy mixer with state of its own, defined here, is registered, built and stepped without a
change to the framework's files: a new architecture (its config, its spec, its tensors), a mixer
that keeps a fixed-size state per request in the slot the cache manager hands out, a run order
that names a layer twice and lets an entry read another entry's cache."""
import numpy as np
import pytest
import torch

import plain_llama as P
import tiny_configs as tc
from fllm_amd.config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.parts.base import INIT_MATRIX, Mixer, StateNeed
from fllm_amd.registry import Architecture, model_spec_from_config, register_architecture, register_part
from fllm_amd.weights import random_tensors

pytestmark = pytest.mark.gpu


class DecayingSum(Mixer):
    """state <- decay * state + x_t ; output_t = W state.  One state vector per request."""

    @classmethod
    def tensor_shapes(cls, spec):
        return {"w": ((spec["hidden_size"], spec["hidden_size"]), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = spec["hidden_size"]
        self.decay = spec["decay"]
        self.w = rt.matrix(weights["w"])

    def state_need(self):
        return StateNeed((self.hidden,), torch.float32)

    def forward(self, ctx, h, residual, binding):
        row = 0
        for rows, start, slot in zip(ctx.seg_rows, ctx.seg_pos_start, ctx.seg_slots):
            state = binding.state[slot]
            if start == 0:
                state.zero_()                       # a new request (or one that is computed again)
            for r in range(row, row + rows):
                state.mul_(self.decay).add_(h[r].float())
                residual[r] += (self.w.float() @ state)
            row += rows


register_part("mixer", "decaying_sum", DecayingSum)


def toy_spec(cfg):
    hidden = cfg["hidden_size"]
    norm = lambda name: PartSpec("rms", {"size": hidden, "eps": 1e-5}, {"weight": name})
    layers = []
    for i in range(2):
        if i == 0:
            mixer = PartSpec("decaying_sum", {"hidden_size": hidden, "decay": cfg["decay"]}, {"w": f"layers.{i}.mix.w"})
        else:
            mixer = PartSpec("attention", {"hidden_size": hidden, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                           "scale": 0.25, "window": None,
                                           "position": {"kind": "rotary", "dims": 16, "theta": 10000.0, "scaling": "none",
                                                        "max_position": 128}},
                             {k: f"layers.{i}.attn.{k}" for k in "qkvo"})
        ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": 96, "activation": "silu"},
                       {k: f"layers.{i}.mlp.{k}" for k in ("gate", "up", "down")})
        layers.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, {"mixer": norm(f"layers.{i}.n1"), "feed_forward": norm(f"layers.{i}.n2")}))
    # the attention layer runs twice (its weights are shared, each run has its own cache), then once
    # more reading the cache of its first run
    order = (RunEntry(0), RunEntry(1), RunEntry(1), RunEntry(1, reads_cache_of=1))
    return ModelSpec("toy-state", hidden, cfg["vocab_size"], 128,
                     PartSpec("table", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "embed"}),
                     tuple(layers), order, norm("final_norm"),
                     PartSpec("linear", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "embed"}))


register_architecture(Architecture("toy-state", ("ToyStateModel",), lambda c: c, toy_spec))
TOY = {"model_type": "toy-state", "hidden_size": 64, "vocab_size": 200, "decay": 0.75}


def plain_toy(w, ids):
    """The same model, whole sequence, float64."""
    x = w["embed"][np.asarray(ids)]
    T = len(ids)

    def mlp(x, i):
        h = P.rms_norm(x, w[f"layers.{i}.n2"], 1e-5)
        return x + P.gated_mlp(h, w[f"layers.{i}.mlp.gate"], w[f"layers.{i}.mlp.up"], w[f"layers.{i}.mlp.down"])

    def attention(x, kv_from=None):
        h = P.rms_norm(x, w["layers.1.n1"], 1e-5)
        cos, sin = P.rope_tables(range(T), 16, 10000.0)
        q = P.apply_rope((h @ w["layers.1.attn.q"].T).reshape(T, 4, 16), cos, sin, 16)
        if kv_from is None:
            k = P.apply_rope((h @ w["layers.1.attn.k"].T).reshape(T, 2, 16), cos, sin, 16)
            v = (h @ w["layers.1.attn.v"].T).reshape(T, 2, 16)
        else:
            k, v = kv_from
        o = P.attention(q, k, v, 0.25).reshape(T, 64) @ w["layers.1.attn.o"].T
        return mlp(x + o, 1), (k, v)

    h = P.rms_norm(x, w["layers.0.n1"], 1e-5)
    state = np.zeros(64)
    out = np.zeros_like(x)
    for t in range(T):
        state = 0.75 * state + h[t]
        out[t] = w["layers.0.mix.w"] @ state
    x = mlp(x + out, 0)
    x, first_cache = attention(x)
    x, _ = attention(x)
    x, _ = attention(x, kv_from=first_cache)
    return P.rms_norm(x, w["final_norm"], 1e-5) @ w["embed"].T


def test_toy_architecture_steps_through_the_engine():
    typed, spec = model_spec_from_config(TOY)
    tensors = random_tensors(spec, 5, torch.float32)
    runner = ModelRunner(spec, tensors, dtype="float32", page_size=16, max_tokens=256, max_requests=4)
    assert not runner.use_graphs                                  # the toy mixer decides on the host: no capture
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].entries == (1, 2)   # two caches, the reader owns none
    assert runner.model.bindings[0].state.shape == (4, 64) and runner.model.bindings[3].writes is False
    w64 = tc.to_float64(tensors)
    a, b = tc.random_ids(50, 200, 1), tc.random_ids(33, 200, 2)
    want_a, want_b = plain_toy(w64, a), plain_toy(w64, b)
    got_a, got_b = [], []
    all_of = lambda toks: list(range(len(toks)))
    # portions of a beside portions and single tokens of b; b arrives later
    got_a.append(runner.step([StepEntry("a", a[:7], all_of(a[:7]))]))
    out = runner.step([StepEntry("a", a[7:30], all_of(a[7:30])), StepEntry("b", b[:20], all_of(b[:20]))])
    got_a.append(out[:23]); got_b.append(out[23:])
    for i in range(20, 33):
        out = runner.step([StepEntry("b", [b[i]], [0]), StepEntry("a", [a[10 + i]], [0])])
        got_b.append(out[:1]); got_a.append(out[1:])
    got_a.append(runner.step([StepEntry("a", a[43:], all_of(a[43:]))]))
    for got, want in ((torch.cat(got_a), want_a), (torch.cat(got_b), want_b)):
        err = np.abs(got.double().cpu().numpy() - want).max()
        assert err <= 3e-5 * np.abs(want).max(), err
    runner.free_request("a")
    # the slot of a is handed out again: the new request starts from a cleared state
    got = runner.step([StepEntry("c", b, all_of(b))])
    assert np.abs(got.double().cpu().numpy() - want_b).max() <= 3e-5 * np.abs(want_b).max()
    runner.cache.check_invariants()
