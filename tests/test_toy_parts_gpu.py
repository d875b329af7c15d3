"""Toy parts, defined here, are registered, built and stepped without a change to the framework's
files.  First a toy mixer with state of its own: a new architecture (its config, its spec, its tensors), a mixer
that keeps a fixed-size state per request in the slot the cache manager hands out, a run order
that names a layer twice and lets an entry read another entry's cache.  Then a feed-forward with
routing and another position encoding."""
import numpy as np
import pytest
import torch

import plain_llama as P
import tiny_configs as tc
from fllm_amd.config.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from fllm_amd.engine import ModelRunner, StepEntry
from fllm_amd.parts.base import INIT_MATRIX, FeedForward, Mixer, Part, StateNeed
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


def plain_toy(w, ids, first_mixer=None):
    """The same model, whole sequence, float64.  `first_mixer`: the output [T, hidden] of another first mixer."""
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
    x = mlp(x + (out if first_mixer is None else first_mixer), 0)
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


def check_shared_beginnings(engine_options):
    """Pages can be shared between requests that begin alike by naming them twice; a mixer's own state has to be copied
    where the requests part.  Further answers to a prompt, and requests behind a known prefix, start from such a copy
    and give the tokens of a request that ran alone.  (Also run on the CPU by tests/test_toy_state_cpu.py.)"""
    from fllm_amd import Engine, SamplingParams
    options = dict(config=TOY, seed=5, dtype="float32", num_blocks=32, max_seqs=4, ctx=128, max_batched_tokens=24)
    options.update(engine_options)
    engine = Engine(**options)
    prompt = tc.random_ids(40, 200, 3)
    alone = engine.generate([prompt], SamplingParams(max_tokens=6))[0]
    rows = engine.stats.prefill_rows
    assert rows == 40
    # three answers: the first one's prompt is cut at its last page boundary (32), the state is copied there, and the
    # other two compute the 8 tokens behind it
    assert engine.generate([prompt], SamplingParams(max_tokens=6, n=3)) == [[alone] * 3]
    assert engine.stats.prefill_rows - rows == 40 + 2 * 8
    engine.runner.cache.check_invariants()
    # sampled answers differ from each other and are what each seed gives alone
    params = SamplingParams(max_tokens=6, n=3, temperature=0.9, seed=11)
    together = engine.generate([prompt], params)[0]
    from dataclasses import replace
    single = [Engine(**options).generate([prompt], replace(params.for_choice(k), n=1))[0] for k in range(3)]
    assert together == single and len({tuple(t) for t in together}) > 1
    # the prefix cache: a second request with the same beginning starts behind the copy
    cached = Engine(prefix_cache=True, **options)
    other = prompt[:35] + tc.random_ids(9, 200, 4)
    want_other = engine.generate([other], SamplingParams(max_tokens=6))[0]
    assert cached.generate([prompt], SamplingParams(max_tokens=6))[0] == alone
    rows = cached.stats.prefill_rows
    assert cached.generate([prompt], SamplingParams(max_tokens=6))[0] == alone
    assert cached.stats.prefill_rows - rows == 8 and cached.stats.prefix_hit_tokens == 32
    rows = cached.stats.prefill_rows
    assert cached.generate([other], SamplingParams(max_tokens=6))[0] == want_other
    assert cached.stats.prefill_rows - rows == 44 - 32          # pages without a copy of the state behind them do not count
    assert cached.generate([prompt, other], SamplingParams(max_tokens=6, n=2)) == [[alone] * 2, [want_other] * 2]
    cached.runner.cache.check_invariants()


def test_toy_state_is_copied_where_requests_part():
    check_shared_beginnings({})


class RunningMean(Mixer):
    """output_t = W mean(x_0 .. x_t): a sum and a count per request, two tensors of different shape and type.  It asks
    for portions that begin on multiples of four tokens, as a mixer whose kernels work on chunks of positions would."""

    @classmethod
    def tensor_shapes(cls, spec):
        return {"w": ((spec["hidden_size"], spec["hidden_size"]), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.hidden = spec["hidden_size"]
        self.w = rt.matrix(weights["w"])

    def state_need(self):
        return {"sum": StateNeed((self.hidden,), torch.float32), "count": StateNeed((1,), torch.int32)}

    def portion_multiple(self):
        return 4

    def forward(self, ctx, h, residual, binding):
        row = 0
        for rows, start, slot in zip(ctx.seg_rows, ctx.seg_pos_start, ctx.seg_slots):
            total, count = binding.state["sum"][slot], binding.state["count"][slot]
            assert rows == 1 or start % 4 == 0, "a portion that begins off a multiple of four"
            assert int(count) == start, "the state is not the one left behind the position before"
            for r in range(row, row + rows):
                total.add_(h[r].float())
                count.add_(1)
                residual[r] += self.w.float() @ (total / count.float())
            row += rows


register_part("mixer", "running_mean", RunningMean)


def mean_spec(cfg):
    spec = toy_spec(cfg)
    mixer = PartSpec("running_mean", {"hidden_size": cfg["hidden_size"]}, {"w": "layers.0.mix.w"})
    first = LayerSpec(spec.layers[0].block, mixer, spec.layers[0].feed_forward, spec.layers[0].norms)
    return ModelSpec("toy-mean", spec.hidden_size, spec.vocab_size, spec.max_position, spec.embedding,
                     (first, spec.layers[1]), spec.run_order, spec.final_norm, spec.head)


register_architecture(Architecture("toy-mean", ("ToyMeanModel",), lambda c: c, mean_spec))
MEAN = {"model_type": "toy-mean", "hidden_size": 64, "vocab_size": 200, "decay": 0.0}


def plain_mean_greedy(w, prompt, count):
    """Greedy tokens of the running-mean model, whole sequences, float64: plain_toy with the mean in place of the
    decaying sum (a decay of 1 and a division by the position)."""
    def logits(ids):
        x = w["embed"][np.asarray(ids)]
        h = P.rms_norm(x, w["layers.0.n1"], 1e-5)
        mean = np.cumsum(h, axis=0) / np.arange(1, len(ids) + 1)[:, None]
        return mean @ w["layers.0.mix.w"].T
    seq, out = list(prompt), []
    for _ in range(count):
        # the rest of the model is plain_toy's: run it with the first mixer's output swapped in
        out.append(int(np.argmax(plain_toy(w, seq, first_mixer=logits(seq))[-1])))
        seq.append(out[-1])
    return out


def check_two_state_tensors(engine_options):
    from fllm_amd import Engine, SamplingParams
    from fllm_amd.engine import StepError
    options = dict(config=MEAN, seed=8, dtype="float32", num_blocks=32, max_seqs=4, ctx=128, max_batched_tokens=22)
    options.update(engine_options)
    engine = Engine(**options)
    state = engine.runner.model.bindings[0].state
    assert set(state) == {"sum", "count"} and state["sum"].shape == (4, 64) and state["count"].dtype == torch.int32
    assert engine.runner.model.portion_multiple == 4 and engine.scheduler.cfg.portion_multiple == 4
    _, spec = model_spec_from_config(MEAN)
    w64 = tc.to_float64(random_tensors(spec, 8, torch.float32))
    prompt = tc.random_ids(45, 200, 6)
    want = plain_mean_greedy(w64, prompt, 5)
    # a budget of 22 tokens a step: the scheduler cuts 20 + 12 (the page boundary at 32, where the state is copied) + 13
    assert engine.generate([prompt], SamplingParams(max_tokens=5, n=3)) == [[want] * 3]
    assert engine.stats.prefill_rows == 45 + 2 * 13
    # snapshots hold both tensors; one of another model is refused
    engine.add_request("r", prompt[:9], SamplingParams(max_tokens=2))
    engine.step()
    sid = engine.scheduler.running[0]
    snapshot = engine.runner.snapshot_state(sid)
    assert sorted(name for _, name, _ in snapshot) == ["count", "sum"] and int(snapshot[0][2] if snapshot[0][1] == "count" else snapshot[1][2]) == 9
    with pytest.raises(ValueError, match="not one of this model"):
        engine.runner.restore_state(sid, snapshot[:1])
    engine.abort_request("r")
    while engine.has_unfinished():
        engine.step()
    # the step function refuses a portion that begins off a multiple
    runner = engine.runner
    runner.step([StepEntry("p", prompt[:6], [])])
    with pytest.raises(StepError, match="multiples of 4"):
        runner.step([StepEntry("p", prompt[6:9], [])])
    runner.step([StepEntry("p", prompt[6:7], [])])             # single tokens go anywhere
    runner.free_request("p")


def test_toy_mixer_with_two_state_tensors_and_portions_on_multiples():
    check_two_state_tensors({})


# ---------------------------------------------------------------------------------------------
# A feed-forward with routing and another position encoding, again without touching the framework
# ---------------------------------------------------------------------------------------------
class TopOneExperts(FeedForward):
    """Router logits in float32; the expert with the largest logit runs, weighted by its softmax
    probability: y = p_e * W2_e relu(W1_e x)."""

    @classmethod
    def tensor_shapes(cls, spec):
        e, h, m = spec["experts"], spec["hidden_size"], spec["intermediate_size"]
        return {"router": ((e, h), INIT_MATRIX), "w1": ((e * m, h), INIT_MATRIX), "w2": ((e * h, m), INIT_MATRIX)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.e, self.h, self.m = spec["experts"], spec["hidden_size"], spec["intermediate_size"]
        self.router = weights["router"].to(rt.device, torch.float32)
        self.w1 = weights["w1"].to(rt.device, torch.float32).view(self.e, self.m, self.h)
        self.w2 = weights["w2"].to(rt.device, torch.float32).view(self.e, self.h, self.m)

    def forward(self, ctx, h, residual):
        x = h.float()
        logits = x @ self.router.T * 40.0          # far apart, so that rounding does not change the choice
        prob, choice = torch.softmax(logits, dim=-1).max(dim=-1)
        for e in range(self.e):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                y = torch.relu(x[rows] @ self.w1[e].T) @ self.w2[e].T
                residual.index_add_(0, rows, y * prob[rows, None])


class SquareRootAngles(Part):
    """Rotation by angles sqrt(position + 1) * (lane + 1) * step on interleaved lane pairs of the first `dims`
    values of a head: what a position part owes the attention mixer is cos/sin tables by position, `dims` and
    `pairing`."""
    role = "position"

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.dims, self.pairing = int(spec["dims"]), 1
        pos = torch.arange(int(spec["max_position"]), dtype=torch.float64)
        lanes = torch.arange(self.dims // 2, dtype=torch.float64)
        phase = torch.sqrt(pos + 1.0)[:, None] * (lanes + 1.0)[None, :] * float(spec["step"])
        self.cos = torch.cos(phase).float().to(rt.device).contiguous()
        self.sin = torch.sin(phase).float().to(rt.device).contiguous()


register_part("feed_forward", "top_one_experts", TopOneExperts)
register_part("position", "sqrt_angles", SquareRootAngles)


def routed_spec(cfg):
    hidden = cfg["hidden_size"]
    norm = lambda name: PartSpec("rms", {"size": hidden, "eps": 1e-6}, {"weight": name})
    layers = []
    for i in range(2):
        position = {"kind": "sqrt_angles", "dims": 8, "step": cfg["step"], "max_position": 128} if i == 0 else None
        mixer = PartSpec("attention", {"hidden_size": hidden, "num_heads": 3, "num_kv_heads": 1, "head_dim": 16, "scale": 0.3,
                                       "window": None, "position": position},
                         {k: f"layers.{i}.attn.{k}" for k in "qkvo"})
        if i == 0:
            ffn = PartSpec("top_one_experts", {"hidden_size": hidden, "intermediate_size": 40, "experts": 3},
                           {k: f"layers.{i}.moe.{k}" for k in ("router", "w1", "w2")})
        else:
            ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": 56, "activation": "silu"},
                           {k: f"layers.{i}.mlp.{k}" for k in ("gate", "up", "down")})
        layers.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, {"mixer": norm(f"layers.{i}.n1"), "feed_forward": norm(f"layers.{i}.n2")}))
    return ModelSpec("toy-routed", hidden, cfg["vocab_size"], 128,
                     PartSpec("table", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "embed"}),
                     tuple(layers), (RunEntry(0), RunEntry(1)), norm("final_norm"),
                     PartSpec("linear", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "head"}))


register_architecture(Architecture("toy-routed", ("ToyRoutedModel",), lambda c: c, routed_spec))
ROUTED = {"model_type": "toy-routed", "hidden_size": 48, "vocab_size": 130, "step": 0.37}


def plain_routed(w, ids):
    """The same model, whole sequence, float64; returns the logits, the experts chosen and the smallest gap between
    the two largest router logits of a token, relative to their size."""
    x = w["embed"][np.asarray(ids)]
    T = len(ids)
    chosen = None
    for i in range(2):
        h = P.rms_norm(x, w[f"layers.{i}.n1"], 1e-6)
        q = (h @ w[f"layers.{i}.attn.q"].T).reshape(T, 3, 16)
        k = (h @ w[f"layers.{i}.attn.k"].T).reshape(T, 1, 16)
        v = (h @ w[f"layers.{i}.attn.v"].T).reshape(T, 1, 16)
        if i == 0:
            phase = np.sqrt(np.arange(T) + 1.0)[:, None] * (np.arange(4) + 1.0)[None, :] * 0.37
            q = P.apply_rope(q, np.cos(phase), np.sin(phase), 8, interleaved=True)
            k = P.apply_rope(k, np.cos(phase), np.sin(phase), 8, interleaved=True)
        x = x + P.attention(q, k, v, 0.3).reshape(T, 48) @ w[f"layers.{i}.attn.o"].T
        h = P.rms_norm(x, w[f"layers.{i}.n2"], 1e-6)
        if i == 0:
            logits = h @ w["layers.0.moe.router"].T * 40.0
            prob = np.exp(logits - logits.max(-1, keepdims=True))
            prob /= prob.sum(-1, keepdims=True)
            chosen = logits.argmax(-1)
            top = np.sort(logits, axis=-1)
            gap = ((top[:, -1] - top[:, -2]) / np.abs(logits).max()).min()
            w1, w2 = w["layers.0.moe.w1"].reshape(3, 40, 48), w["layers.0.moe.w2"].reshape(3, 48, 40)
            y = np.stack([np.maximum(h[t] @ w1[e].T, 0.0) @ w2[e].T * prob[t, e] for t, e in enumerate(chosen)])
            x = x + y
        else:
            x = x + P.gated_mlp(h, w["layers.1.mlp.gate"], w["layers.1.mlp.up"], w["layers.1.mlp.down"])
    return P.rms_norm(x, w["final_norm"], 1e-6) @ w["head"].T, chosen, gap


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_toy_routed_feed_forward_and_position_encoding(dtype, tol):
    """A feed-forward that routes every token to one of three experts and a position encoding with its own angles,
    interleaved pairs and fewer lanes than the head has, beside a layer of attention without positions and the
    framework's own feed-forward; portions, single tokens and a second request, against the whole sequence."""
    typed, spec = model_spec_from_config(ROUTED)
    tensors = random_tensors(spec, 52, torch.float32 if dtype == "float32" else torch.bfloat16)   # a seed without near-ties in the router
    runner = ModelRunner(spec, tensors, dtype=dtype, page_size=16, max_tokens=192, max_requests=2)
    w64 = tc.to_float64(tensors)
    a, b = tc.random_ids(61, 130, 7), tc.random_ids(40, 130, 8)
    (want_a, chosen_a, gap_a), (want_b, chosen_b, gap_b) = plain_routed(w64, a), plain_routed(w64, b)
    assert len(set(chosen_a.tolist())) == 3 and len(set(chosen_b.tolist())) >= 2     # the router does route
    assert min(gap_a, gap_b) > 0.02      # no token so close to a tie that bfloat16 rounding could choose otherwise
    all_of = lambda toks: list(range(len(toks)))
    got_a, got_b = [], []
    got_a.append(runner.step([StepEntry("a", a[:19], all_of(a[:19]))]))
    out = runner.step([StepEntry("b", b[:2], all_of(b[:2])), StepEntry("a", a[19:50], all_of(a[19:50]))])
    got_b.append(out[:2]); got_a.append(out[2:])
    out = runner.step([StepEntry("b", b[2:], all_of(b[2:])), StepEntry("a", [a[50]], [0])])
    got_b.append(out[:38]); got_a.append(out[38:])
    for i in range(51, 61):
        got_a.append(runner.step([StepEntry("a", [a[i]], [0])]))
    for got, want in ((torch.cat(got_a), want_a), (torch.cat(got_b), want_b)):
        err = np.abs(got.double().cpu().numpy() - want).max()
        assert err <= tol * np.abs(want).max(), err
    runner.cache.check_invariants()


# ---------------------------------------------------------------------------------------------
# A norm of another kind, layers without a feed-forward, and a state that the mixer never clears itself
# ---------------------------------------------------------------------------------------------
from fllm_amd.parts.base import INIT_NORM, Norm  # noqa: E402


class PlusOneNorm(Norm):
    """y = x * rsqrt(mean(x^2) + eps) * (1 + w): the weight is stored as a distance from one.  It says what a kernel
    needs to apply it (`fused_prologue`), and so gets the decode kernels that norm their input on the way in."""

    @classmethod
    def tensor_shapes(cls, spec):
        return {"weight": ((spec["size"],), INIT_NORM)}

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.size, self.eps = int(spec["size"]), float(spec["eps"])
        self.scale = (rt.vector(weights["weight"]) + 1.0).contiguous()

    def forward(self, ctx, x, out=None, rows=None):
        count = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty((count, self.size)) if out is None else out
        return self.rt.ops.rmsnorm(x, self.scale, self.eps, out, rows=rows)

    def fused_prologue(self):
        return self.scale, self.eps


class TrustingSum(DecayingSum):
    """The decaying sum again, but it never clears its state: it relies on the step function handing a request's
    slot over filled with zeros."""

    def forward(self, ctx, h, residual, binding):
        row = 0
        for rows, slot in zip(ctx.seg_rows, ctx.seg_slots):
            state = binding.state[slot]
            for r in range(row, row + rows):
                state.mul_(self.decay).add_(h[r].float())
                residual[r] += (self.w.float() @ state)
            row += rows


register_part("norm", "rms_plus_one", PlusOneNorm)
register_part("mixer", "trusting_sum", TrustingSum)


def bare_spec(cfg):
    hidden = cfg["hidden_size"]
    norm = lambda name: PartSpec("rms_plus_one", {"size": hidden, "eps": 1e-5}, {"weight": name})
    attention = lambda i: PartSpec("attention", {"hidden_size": hidden, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                                 "scale": 0.25, "window": None,
                                                 "position": {"kind": "rotary", "dims": 16, "theta": 10000.0, "scaling": "none",
                                                              "pairing": "interleaved", "max_position": 128}},
                                   {k: f"layers.{i}.attn.{k}" for k in "qkvo"})
    layers = [LayerSpec(PartSpec("prenorm"), attention(0), norms={"mixer": norm("layers.0.n1")})]      # no feed-forward
    if cfg["stateful"]:
        layers.append(LayerSpec(PartSpec("prenorm"), PartSpec("trusting_sum", {"hidden_size": hidden, "decay": 0.5},
                                                              {"w": "layers.1.mix.w"}), norms={"mixer": norm("layers.1.n1")}))
    else:
        ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": 96, "activation": "silu"},
                       {k: f"layers.1.mlp.{k}" for k in ("gate", "up", "down")})
        layers.append(LayerSpec(PartSpec("prenorm"), attention(1), ffn,
                                {"mixer": norm("layers.1.n1"), "feed_forward": norm("layers.1.n2")}))
    return ModelSpec("toy-bare", hidden, cfg["vocab_size"], 128,
                     PartSpec("table", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "embed"}),
                     tuple(layers), (RunEntry(0), RunEntry(1)), norm("final_norm"),
                     PartSpec("linear", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "head"}))


register_architecture(Architecture("toy-bare", ("ToyBareModel",), lambda c: c, bare_spec))


def plain_bare(w, ids, stateful):
    x = w["embed"][np.asarray(ids)]
    T = len(ids)
    norm = lambda x, name: P.rms_norm(x, 1.0 + w[name], 1e-5)
    cos, sin = P.rope_tables(range(T), 16, 10000.0)

    def attention(x, i):
        h = norm(x, f"layers.{i}.n1")
        q = P.apply_rope((h @ w[f"layers.{i}.attn.q"].T).reshape(T, 4, 16), cos, sin, 16, interleaved=True)
        k = P.apply_rope((h @ w[f"layers.{i}.attn.k"].T).reshape(T, 2, 16), cos, sin, 16, interleaved=True)
        v = (h @ w[f"layers.{i}.attn.v"].T).reshape(T, 2, 16)
        return x + P.attention(q, k, v, 0.25).reshape(T, 64) @ w[f"layers.{i}.attn.o"].T

    x = attention(x, 0)
    if stateful:
        h = norm(x, "layers.1.n1")
        state = np.zeros(64)
        out = np.zeros_like(x)
        for t in range(T):
            state = 0.5 * state + h[t]
            out[t] = w["layers.1.mix.w"] @ state
        x = x + out
    else:
        x = attention(x, 1)
        h = norm(x, "layers.1.n2")
        x = x + P.gated_mlp(h, w["layers.1.mlp.gate"], w["layers.1.mlp.up"], w["layers.1.mlp.down"])
    return norm(x, "final_norm") @ w["head"].T


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 1.5e-2)])
def test_toy_norm_keeps_the_fused_decode_kernels_and_a_layer_may_lack_a_feed_forward(dtype, tol):
    cfg = {"model_type": "toy-bare", "hidden_size": 64, "vocab_size": 150, "stateful": False}
    _, spec = model_spec_from_config(cfg)
    tensors = {k: v.float() for k, v in random_tensors(spec, 23, torch.bfloat16).items()}
    runner = ModelRunner(spec, tensors, dtype=dtype, page_size=16, max_tokens=256, max_requests=4)
    assert runner.use_graphs and runner.model.blocks[0].feed_forward is None
    calls = {"norm_qkv_rope_store": 0, "norm_gate_up_swiglu": 0, "linear_add_prepare": 0}
    fed = {"norm_qkv_rope_store": 0, "norm_gate_up_swiglu": 0}       # calls that got a norm prepared by the sum before
    for name in calls:
        def counted(*args, _fn=getattr(runner.rt.ops, name), _name=name, **kw):
            calls[_name] += 1
            if kw.get("prepared") is not None:
                fed[_name] += 1
            return _fn(*args, **kw)
        setattr(runner.rt.ops, name, counted)
    try:
        w64 = tc.to_float64(tensors)
        a, b = tc.random_ids(40, 150, 3), tc.random_ids(25, 150, 4)
        want_a, want_b = plain_bare(w64, a, False), plain_bare(w64, b, False)
        all_of = lambda toks: list(range(len(toks)))
        got_a = [runner.step([StepEntry("a", a[:30], all_of(a[:30]))])]
        got_b = [runner.step([StepEntry("b", b[:20], all_of(b[:20]))])]
        for i in range(5):      # a step's logits are valid until the next step: decode graphs write them in place
            out = runner.step([StepEntry("a", [a[30 + i]], [0]), StepEntry("b", [b[20 + i]], [0])]).clone()
            got_a.append(out[:1]); got_b.append(out[1:])
        for i in range(35, 40):
            got_a.append(runner.step([StepEntry("a", [a[i]], [0])]).clone())
    finally:
        for name in calls:
            delattr(runner.rt.ops, name)
    for got, want in ((torch.cat(got_a), want_a), (torch.cat(got_b), want_b)):
        err = np.abs(got.double().cpu().numpy() - want).max()
        assert err <= tol * np.abs(want).max(), err
    if dtype == "bfloat16":      # the decode steps went through the kernels that norm on the way in, and through graphs
        assert calls["norm_qkv_rope_store"] >= 2 and calls["norm_gate_up_swiglu"] >= 1 and runner.graph_replays >= 8
        # the toy norm says what it multiplies by, so the sums before it prepare it: every norm but a step's first one
        # comes prepared (a layer without a feed-forward prepares the first norm of the layer after)
        assert calls["linear_add_prepare"] > 0 and fed["norm_qkv_rope_store"] + fed["norm_gate_up_swiglu"] == calls["linear_add_prepare"]
        assert 2 * fed["norm_qkv_rope_store"] == calls["norm_qkv_rope_store"] and fed["norm_gate_up_swiglu"] == calls["norm_gate_up_swiglu"]
    else:
        assert calls == {"norm_qkv_rope_store": 0, "norm_gate_up_swiglu": 0, "linear_add_prepare": 0}


def test_state_slot_is_handed_over_cleared():
    """A mixer that never clears its state: a request's first step finds zeros, also in a slot that another request
    used before and also when the same request is freed and fed again."""
    cfg = {"model_type": "toy-bare", "hidden_size": 64, "vocab_size": 150, "stateful": True}
    _, spec = model_spec_from_config(cfg)
    tensors = random_tensors(spec, 29, torch.float32)
    runner = ModelRunner(spec, tensors, dtype="float32", page_size=16, max_tokens=256, max_requests=2)
    w64 = tc.to_float64(tensors)
    a, b = tc.random_ids(30, 150, 5), tc.random_ids(21, 150, 6)
    want_a, want_b = plain_bare(w64, a, True), plain_bare(w64, b, True)
    all_of = lambda toks: list(range(len(toks)))
    close = lambda got, want: np.abs(got.double().cpu().numpy() - want).max() <= 3e-5 * np.abs(want).max()
    first = torch.cat([runner.step([StepEntry("a", a[:11], all_of(a[:11]))]), runner.step([StepEntry("a", a[11:], all_of(a[11:]))])])
    assert close(first, want_a)
    slot = runner.cache.slot("a")
    runner.free_request("a")
    assert close(runner.step([StepEntry("b", b, all_of(b))]), want_b) and runner.cache.slot("b") == slot
    runner.free_request("b")
    half = runner.step([StepEntry("a", a[:15], all_of(a[:15]))])            # given up half way ...
    runner.free_request("a")
    again = runner.step([StepEntry("a", a, all_of(a))])                    # ... and fed again from its first token
    assert close(half, want_a[:15]) and close(again, want_a)


# ---------------------------------------------------------------------------------------------
# A position encoding that rotates nothing and biases every score by the distance to the key
# ---------------------------------------------------------------------------------------------
class DistanceSlopes(Part):
    """score(row, key) += slope[head] * (key position - row position), slope[head] = -base ** -(head + 1): what
    such a part owes the attention mixer is `score_slopes` (float32 [heads] on the device) beside rotary arguments
    that rotate nothing (`dims` 0, empty tables)."""
    role = "position"

    def __init__(self, spec, weights, rt):
        super().__init__(spec, weights, rt)
        self.dims, self.pairing = 0, 1
        self.cos = self.sin = torch.zeros((1, 0), dtype=torch.float32, device=rt.device)
        slopes = [float(spec["base"]) ** -(h + 1) for h in range(int(spec["heads"]))]
        self.score_slopes = torch.tensor(slopes, dtype=torch.float32, device=rt.device)


register_part("position", "distance_slopes", DistanceSlopes)


def slopes_spec(cfg):
    hidden = cfg["hidden_size"]
    norm = lambda name: PartSpec("rms", {"size": hidden, "eps": 1e-6}, {"weight": name})
    layers = []
    for i, window in enumerate((None, 24)):
        mixer = PartSpec("attention", {"hidden_size": hidden, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16, "scale": 0.25,
                                       "window": window, "position": {"kind": "distance_slopes", "base": cfg["base"], "heads": 4}},
                         {k: f"layers.{i}.attn.{k}" for k in "qkvo"})
        ffn = PartSpec("gated_mlp", {"hidden_size": hidden, "intermediate_size": 56, "activation": "silu"},
                       {k: f"layers.{i}.mlp.{k}" for k in ("gate", "up", "down")})
        layers.append(LayerSpec(PartSpec("prenorm"), mixer, ffn, {"mixer": norm(f"layers.{i}.n1"), "feed_forward": norm(f"layers.{i}.n2")}))
    return ModelSpec("toy-slopes", hidden, cfg["vocab_size"], 256,
                     PartSpec("table", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "embed"}),
                     tuple(layers), (RunEntry(0), RunEntry(1)), norm("final_norm"),
                     PartSpec("linear", {"vocab_size": cfg["vocab_size"], "hidden_size": hidden}, {"weight": "head"}))


register_architecture(Architecture("toy-slopes", ("ToySlopesModel",), lambda c: c, slopes_spec))
SLOPES = {"model_type": "toy-slopes", "hidden_size": 40, "vocab_size": 90, "base": 1.6}


def biased_attention(q, k, v, scale, slopes, window=None):
    """P.attention with slopes[h] * (key - row) added to every score (keys behind the row: a negative distance)."""
    T, heads, d = q.shape
    group = heads // k.shape[1]
    out = np.zeros((T, heads, d))
    for r in range(T):
        start = 0 if window is None else max(0, r + 1 - window)
        for h in range(heads):
            s = (k[start:r + 1, h // group] @ q[r, h]) * scale + slopes[h] * (np.arange(start, r + 1) - r)
            e = np.exp(s - s.max())
            out[r, h] = (e / e.sum()) @ v[start:r + 1, h // group]
    return out


def plain_slopes(w, ids, slopes):
    x = w["embed"][np.asarray(ids)]
    T = len(ids)
    for i, window in enumerate((None, 24)):
        h = P.rms_norm(x, w[f"layers.{i}.n1"], 1e-6)
        q = (h @ w[f"layers.{i}.attn.q"].T).reshape(T, 4, 16)
        k = (h @ w[f"layers.{i}.attn.k"].T).reshape(T, 2, 16)
        v = (h @ w[f"layers.{i}.attn.v"].T).reshape(T, 2, 16)
        x = x + biased_attention(q, k, v, 0.25, slopes, window).reshape(T, 64) @ w[f"layers.{i}.attn.o"].T
        h = P.rms_norm(x, w[f"layers.{i}.n2"], 1e-6)
        x = x + P.gated_mlp(h, w[f"layers.{i}.mlp.gate"], w[f"layers.{i}.mlp.up"], w[f"layers.{i}.mlp.down"])
    return P.rms_norm(x, w["final_norm"], 1e-6) @ w["head"].T


@pytest.mark.parametrize("dtype,tol", [("float32", 3e-5), ("bfloat16", 4e-2)])
def test_toy_position_encoding_that_biases_scores(dtype, tol):
    """A position part that hands the attention mixer a slope per head instead of angles: scores fall off with the
    distance to the key, in a layer with all keys and in one with a window; portions, single tokens and a second
    request against the whole sequence.  The plain function equals plain attention at slopes of zero, and the bias
    matters: without it the logits are far from the ones wanted."""
    rng = np.random.default_rng(3)
    q, k, v = rng.standard_normal((9, 4, 16)), rng.standard_normal((9, 2, 16)), rng.standard_normal((9, 2, 16))
    assert np.allclose(biased_attention(q, k, v, 0.25, np.zeros(4), 5), P.attention(q, k, v, 0.25, 5), atol=1e-12)
    typed, spec = model_spec_from_config(SLOPES)
    tensors = random_tensors(spec, 21, torch.float32 if dtype == "float32" else torch.bfloat16)
    for name in tensors:                       # larger q and k, so that scores and their bias are of one size
        if name.endswith("attn.q") or name.endswith("attn.k"):
            tensors[name] = tensors[name] * 8
    runner = ModelRunner(spec, tensors, dtype=dtype, page_size=16, max_tokens=256, max_requests=2)
    w64 = tc.to_float64(tensors)
    slopes = np.array([1.6 ** -(h + 1) for h in range(4)])
    a, b = tc.random_ids(70, 90, 5), tc.random_ids(33, 90, 6)
    want_a, want_b = plain_slopes(w64, a, slopes), plain_slopes(w64, b, slopes)
    assert np.abs(plain_slopes(w64, a, np.zeros(4)) - want_a).max() > 0.05 * np.abs(want_a).max()
    all_of = lambda toks: list(range(len(toks)))
    got_a, got_b = [], []
    got_a.append(runner.step([StepEntry("a", a[:23], all_of(a[:23]))]))
    out = runner.step([StepEntry("b", b[:2], all_of(b[:2])), StepEntry("a", a[23:60], all_of(a[23:60]))])
    got_b.append(out[:2]); got_a.append(out[2:])
    out = runner.step([StepEntry("b", b[2:], all_of(b[2:])), StepEntry("a", [a[60]], [0])])
    got_b.append(out[:31]); got_a.append(out[31:])
    for i in range(61, 70):
        got_a.append(runner.step([StepEntry("a", [a[i]], [0])]).clone())
    for got, want in ((torch.cat(got_a), want_a), (torch.cat(got_b), want_b)):
        err = np.abs(got.double().cpu().numpy() - want).max()
        assert err <= tol * np.abs(want).max(), err
    runner.cache.check_invariants()
