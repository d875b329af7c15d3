"""Pins the plain implementation by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place, a head
mapped to the wrong group) fails it."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
import tiny_configs as tc
from fllm_amd.registry import model_spec_from_config
from fllm_amd.weights import random_tensors


def rng(seed):
    return np.random.default_rng(seed)


# ---- RMSNorm ---------------------------------------------------------------------------------
def test_rms_norm_reduces_to_unit_rms_and_matches_the_library():
    x = rng(1).normal(size=(5, 48)) * 3
    w = 1 + 0.1 * rng(2).normal(size=48)
    y = P.rms_norm(x, w, 1e-12)
    assert np.allclose(y / w, x / np.linalg.norm(x, axis=-1, keepdims=True) * math.sqrt(48), rtol=1e-9)
    lib = F.rms_norm(torch.tensor(x), (48,), torch.tensor(w), eps=1e-5).numpy()
    assert np.allclose(P.rms_norm(x, w, 1e-5), lib, rtol=1e-12)
    assert np.allclose(P.rms_norm(7.0 * x, w, 1e-12), y, rtol=1e-9)              # scale invariance
    assert not np.allclose(P.rms_norm(x, w, 1e-5), (x - x.mean(-1, keepdims=True)) / x.std(-1, keepdims=True) * w)


def test_rms_norm_eps_is_inside_the_root():
    x = np.full((1, 4), 1e-3)
    assert np.allclose(P.rms_norm(x, np.ones(4), 1e-2), x / math.sqrt(1e-6 + 1e-2))


# ---- rotary ----------------------------------------------------------------------------------
def test_rope_tables_reference_vectors():
    """rust/engine/src/rope.rs:134-142: position 0 is the identity, lane 1 of 8 dims at base
    10000 turns at frequency 0.1."""
    cos, sin = P.rope_tables([0, 1, 2], 8, 10000.0)
    assert cos.shape == (3, 4) and np.all(cos[0] == 1.0) and np.all(sin[0] == 0.0)
    assert abs(sin[1, 0] - math.sin(1.0)) < 1e-7 and abs(sin[1, 1] - math.sin(0.1)) < 1e-7


def test_linear_scaling_divides_the_position():
    """rust/engine/src/rope.rs:144-151."""
    plain = P.rope_tables(range(9), 8, 10000.0)[1]
    linear = P.rope_tables(range(9), 8, 10000.0, "linear", {"factor": 4.0})[1]
    assert np.allclose(linear[8], plain[2], atol=1e-6)


def test_yarn_reference_vector():
    """rust/engine/src/rope.rs:153-175: 8 dims, base 10000, factor 4, original context 64, beta 32 / 1, truncated:
    the fastest lane keeps its angle and only grows by 1 + 0.1 ln 4, the slowest turns a quarter as far."""
    yarn = {"factor": 4.0, "original_max_position_embeddings": 64}
    pc, ps = P.rope_tables(range(40), 8, 10000.0)
    yc, ys = P.rope_tables(range(40), 8, 10000.0, "yarn", yarn)
    magnitude = 1.0 + 0.1 * math.log(4.0)
    angle = lambda c, s, p, l: math.atan2(s[p, l], c[p, l])
    assert abs(angle(yc, ys, 30, 0) - angle(pc, ps, 30, 0)) < 1e-5
    assert abs(math.hypot(yc[30, 0], ys[30, 0]) - magnitude) < 1e-5
    assert abs(angle(yc, ys, 30, 3) - angle(pc, ps, 30, 3) / 4.0) < 1e-5
    # a wrong direction of the ramp would interpolate the fast lane instead: 30 rad / 4 is another angle
    assert abs(angle(yc, ys, 30, 0) - math.atan2(math.sin(7.5), math.cos(7.5))) > 0.1


def test_yarn_special_cases():
    plain = P.rope_tables(range(50), 16, 10000.0)
    # factor 1: both angles are the same and ln 1 = 0: plain rotary
    one = P.rope_tables(range(50), 16, 10000.0, "yarn", {"factor": 1.0, "original_max_position_embeddings": 32})
    assert np.allclose(one[0], plain[0], atol=1e-6) and np.allclose(one[1], plain[1], atol=1e-6)
    # no extrapolation at all: linear scaling times the attention factor alone (rope.rs:87-91, :97-101)
    lin = P.rope_tables(range(50), 16, 10000.0, "linear", {"factor": 4.0})
    flat = P.rope_tables(range(50), 16, 10000.0, "yarn", {"factor": 4.0, "original_max_position_embeddings": 32,
                                                           "extrapolation_factor": 0.0})
    assert np.allclose(flat[0], lin[0], atol=1e-6) and np.allclose(flat[1], lin[1], atol=1e-6)
    # the checkpoint's attention_factor IS the magnitude: it replaces 1 + 0.1 ln(factor) (plan.rs:1460-1476)
    given = P.rope_tables(range(50), 16, 10000.0, "yarn", {"factor": 4.0, "original_max_position_embeddings": 32,
                                                            "attention_factor": 1.25})
    assert np.allclose(np.hypot(given[0], given[1]), 1.25, atol=1e-6)
    # the pair of mscales gives the quotient of their magnitudes
    pair = P.rope_tables(range(50), 16, 10000.0, "yarn", {"factor": 4.0, "original_max_position_embeddings": 32,
                                                           "mscale": 1.0, "mscale_all_dim": 0.5})
    want = (1 + 0.1 * math.log(4.0)) / (1 + 0.05 * math.log(4.0))
    assert np.allclose(np.hypot(pair[0], pair[1]), want, atol=1e-6)
    # lanes between the two correction dimensions lie between both angles: 64 dims, original 2048: low 8, high 21
    y = P.yarn_values({"factor": 8.0, "original_max_position_embeddings": 2048})
    assert (y["beta_fast"], y["beta_slow"], y["truncate"], float(y["attention"])) == (32.0, 1.0, True, 1.0)
    yc, ys = P.rope_tables([100], 64, 10000.0, "yarn", {"factor": 8.0, "original_max_position_embeddings": 2048})
    pc, ps = P.rope_tables([100], 64, 10000.0)
    turn = lambda c, s, l: math.atan2(s[0, l], c[0, l])
    inv = lambda l: 10000.0 ** (-2.0 * l / 64)
    for lane in (0, 5, 8):
        assert abs(turn(yc, ys, lane) - turn(pc, ps, lane)) < 1e-4               # up to low: untouched
    for lane in (21, 25, 31):
        assert abs(turn(yc, ys, lane) - 100 * inv(lane) / 8.0) < 1e-5            # from high on: position / 8
    mid = 100 * inv(14)
    assert mid / 8.0 + 0.1 < turn(yc, ys, 14) < mid - 0.1 < math.pi              # between: between
    want = mid / 8.0 * (1 - (1 - 6 / 13)) + mid * (1 - 6 / 13)                   # the ramp is a straight line in the lane
    assert abs(turn(yc, ys, 14) - want) < 1e-5


def test_longrope_chooses_factors_by_the_context():
    """rust/engine/src/rope.rs:30-36, :58-66; the magnitude of rust/checkpoint/src/plan.rs:1533-1538."""
    short = [1.0, 1.5, 2.0, 2.5]
    long = [1.0, 3.0, 6.0, 9.0]
    s = {"short_factor": short, "long_factor": long, "original_max_position_embeddings": 64}
    plain = P.rope_tables(range(20), 8, 10000.0)
    angle = lambda c, s_, p, l: math.atan2(s_[p, l], c[p, l])
    within = P.rope_tables(range(20), 8, 10000.0, "longrope", s, context=64, model_context=256)
    beyond = P.rope_tables(range(20), 8, 10000.0, "longrope", s, context=65, model_context=256)
    magnitude = math.sqrt(1.0 + math.log(4.0) / math.log(64.0))
    for tables, factors in ((within, short), (beyond, long)):
        assert np.allclose(np.hypot(*tables), magnitude, atol=1e-6)
        for lane in range(4):
            assert abs(angle(*tables, 12, lane) - angle(*plain, 12, lane) / factors[lane]) < 1e-5
    # a model that is no longer than its original context: magnitude 1; with all factors 1 plain rotary
    ones = {"short_factor": [1.0] * 4, "long_factor": [1.0] * 4, "original_max_position_embeddings": 64}
    same = P.rope_tables(range(20), 8, 10000.0, "su", ones, context=64, model_context=64)
    assert np.allclose(same[0], plain[0], atol=1e-7) and np.allclose(same[1], plain[1], atol=1e-7)
    fixed = P.rope_tables(range(20), 8, 10000.0, "longrope", dict(ones, attention_factor=1.5), context=64, model_context=64)
    assert np.allclose(np.hypot(*fixed), 1.5, atol=1e-6)


def test_dynamic_alpha_only_changes_the_base():
    """rust/checkpoint/src/plan.rs:1339-1343."""
    cfg = {"hidden_size": 64, "num_attention_heads": 4, "num_hidden_layers": 1, "intermediate_size": 8, "head_dim": 16,
           "rope_theta": 10000.0, "rope_scaling": {"rope_type": "dynamic", "alpha": 4.0, "factor": 2.0}}
    sizes = P.read_sizes(cfg)
    assert sizes["rope_kind"] == "default" and abs(sizes["theta"] - 10000.0 * 4.0 ** (16 / 14)) < 1e-6


def test_llama3_divisors_reference_vector():
    """rust/checkpoint/src/plan.rs:3219-3232: head_dim 16, theta 5e5, factor 8, low 1, high 4,
    original 8192: 8 divisors, the first 1.0, the last 8.0."""
    d = P.llama3_divisors(16, 500000.0, 8.0, 1.0, 4.0, 8192.0)
    assert len(d) == 8 and d[0] == 1.0 and d[7] == 8.0
    assert np.all(np.diff(d) >= 0) and np.all((d >= 1.0) & (d <= 8.0))
    assert 1.0 < d[4] < 8.0                                      # a lane in the smooth band
    assert np.all(P.llama3_divisors(16, 500000.0, 8.0, 1.0, 4.0, 1e12) == 1.0)    # huge original context: plain rotary


def test_rotation_keeps_norms_and_depends_on_distance_only():
    q = rng(3).normal(size=(1, 2, 16))
    k = rng(4).normal(size=(1, 2, 16))

    def dot(pq, pk, **kw):
        cq, sq = P.rope_tables([pq], 16, 10000.0)
        ck, sk = P.rope_tables([pk], 16, 10000.0)
        return (P.apply_rope(q, cq, sq, 16, **kw) * P.apply_rope(k, ck, sk, 16, **kw)).sum(-1)

    c, s = P.rope_tables([5], 16, 10000.0)
    assert np.allclose(np.linalg.norm(P.apply_rope(q, c, s, 16), axis=-1), np.linalg.norm(q, axis=-1))
    assert np.allclose(dot(3, 1), dot(12, 10), atol=1e-5) and np.allclose(dot(0, 0), (q * k).sum(-1))
    assert not np.allclose(dot(3, 1), dot(1, 3), atol=1e-3)      # the sign of the rotation matters
    # a query ahead of its key by t turns lane 0 by +t radians: <R(t)q, R(0)k> = cos t for q = k = e_0
    e = np.zeros((1, 1, 16))
    e[0, 0, 0] = 1.0
    c2, s2 = P.rope_tables([2], 16, 10000.0)
    r = P.apply_rope(e, c2, s2, 16)
    assert abs(r[0, 0, 0] - math.cos(2.0)) < 1e-6 and abs(r[0, 0, 8] - math.sin(2.0)) < 1e-6   # pairs (l, l + 8)


def test_half_pairing_equals_the_reference_interleaved_pairing_on_permuted_rows():
    """rust/checkpoint/src/convert.rs:2713-2745: the importer moves row src < half to 2*src and
    row src >= half to 2*(src - half) + 1, then rotates pairs (2l, 2l+1)."""
    d = 16
    x = rng(5).normal(size=(3, 2, d))
    cos, sin = P.rope_tables([0, 7, 31], d, 10000.0)
    dest = np.array([2 * s if s < d // 2 else 2 * (s - d // 2) + 1 for s in range(d)])
    permuted = np.empty_like(x)
    permuted[:, :, dest] = x
    a = P.apply_rope(x, cos, sin, d)
    b = P.apply_rope(permuted, cos, sin, d, interleaved=True)
    assert np.allclose(a, b[:, :, dest])


def test_partial_rotary_leaves_the_rest_alone():
    x = rng(6).normal(size=(2, 1, 16))
    cos, sin = P.rope_tables([3, 4], 8, 10000.0)
    y = P.apply_rope(x, cos, sin, 8)
    assert np.array_equal(y[:, :, 8:], x[:, :, 8:]) and not np.allclose(y[:, :, :8], x[:, :, :8])


# ---- attention -------------------------------------------------------------------------------
def test_attention_reduces_to_the_library_routine():
    T, heads, kv_heads, d = 9, 6, 2, 8
    q, k, v = (rng(s).normal(size=(T, h, d)) for s, h in ((7, heads), (8, kv_heads), (9, kv_heads)))
    got = P.attention(q, k, v, 1 / math.sqrt(d))
    tq, tk, tv = (torch.tensor(a).transpose(0, 1) for a in (q, k, v))
    lib = F.scaled_dot_product_attention(tq, tk.repeat_interleave(3, 0), tv.repeat_interleave(3, 0), is_causal=True)
    assert np.allclose(got, lib.transpose(0, 1).numpy(), atol=1e-12)
    wrong_groups = F.scaled_dot_product_attention(tq, tk.repeat(3, 1, 1), tv.repeat(3, 1, 1), is_causal=True)
    assert not np.allclose(got, wrong_groups.transpose(0, 1).numpy(), atol=1e-3)       # h -> h // group, not h % kv_heads


def test_attention_special_cases():
    d = 8
    v = rng(10).normal(size=(5, 1, d))
    q = rng(11).normal(size=(5, 2, d))
    one = P.attention(q[:1], np.zeros((1, 1, d)), v[:1], 1.0)
    assert np.allclose(one[0, 0], v[0, 0])                                             # a single token returns its value
    flat = P.attention(q, np.zeros((5, 1, d)), v, 1.0)
    assert np.allclose(flat[4, 1], v[:, 0].mean(0)) and np.allclose(flat[2, 0], v[:3, 0].mean(0))   # equal scores: the mean


def test_attention_window_counts_the_token_itself():
    T, d, w = 12, 8, 4
    q, k, v = (rng(s).normal(size=(T, 1, d)) for s in (12, 13, 14))
    got = P.attention(q, k, v, 0.5, window=w)
    mask = torch.tensor([[0 <= r - c < w for c in range(T)] for r in range(T)])
    lib = F.scaled_dot_product_attention(*(torch.tensor(a).transpose(0, 1) for a in (q, k, v)), attn_mask=mask, scale=0.5)
    assert np.allclose(got, lib.transpose(0, 1).numpy(), atol=1e-12)
    assert np.allclose(P.attention(q, k, v, 0.5, window=T), P.attention(q, k, v, 0.5))


# ---- feed-forward ----------------------------------------------------------------------------
def test_silu_and_gated_mlp():
    x = np.array([0.0, 40.0, -40.0, 1.5])
    assert P.silu(x)[0] == 0.0 and abs(P.silu(x)[1] - 40.0) < 1e-12 and abs(P.silu(x)[2]) < 1e-12
    assert np.allclose(P.silu(x), F.silu(torch.tensor(x)).numpy())
    h, i = 6, 10
    xs, g, u, dn = rng(15).normal(size=(3, h)), rng(16).normal(size=(i, h)), rng(17).normal(size=(i, h)), rng(18).normal(size=(h, i))
    want = (F.silu(torch.tensor(xs @ g.T)) * torch.tensor(xs @ u.T)).numpy() @ dn.T
    assert np.allclose(P.gated_mlp(xs, g, u, dn), want)
    assert not np.allclose(P.gated_mlp(xs, u, g, dn), want)                            # the activation sits on the gate


# ---- whole model -----------------------------------------------------------------------------
@pytest.fixture(scope="module")
def weights():
    out = {}
    for name, cfg in tc.CONFIGS.items():
        _, spec = model_spec_from_config(cfg)
        out[name] = tc.to_float64(random_tensors(spec, 21, torch.float32, with_optional=(name == "C")))
    return out


@pytest.mark.parametrize("name", ["A", "B", "C", "F", "G"])
def test_a_shift_of_all_positions_changes_nothing(weights, name):
    """Rotary attention sees distances only (also with per-lane, linear, yarn or longrope scaling)."""
    cfg = tc.CONFIGS[name]
    ids = tc.random_ids(20, cfg["vocab_size"], 1)
    a = P.forward(cfg, weights[name], ids)
    b = P.forward(cfg, weights[name], ids, first_position=37)
    assert np.allclose(a, b, atol=2e-4 * np.abs(a).max())     # float32 phases: the tables differ in the last bits


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_causality_and_the_head(weights, name):
    cfg = tc.CONFIGS[name]
    ids = tc.random_ids(24, cfg["vocab_size"], 2)
    full = P.forward(cfg, weights[name], ids)
    assert full.shape == (24, cfg["vocab_size"])
    assert np.allclose(P.forward(cfg, weights[name], ids[:10]), full[:10], atol=1e-12)       # later tokens change nothing
    other = list(ids)
    other[3] = (other[3] + 1) % cfg["vocab_size"]
    changed = P.forward(cfg, weights[name], other)
    assert np.allclose(changed[:3], full[:3], atol=1e-12) and not np.allclose(changed[3:], full[3:], atol=1e-6)


def test_tied_head_is_the_embedding_table(weights):
    cfg = tc.TINY_B
    w = dict(weights["B"])
    ids = tc.random_ids(6, 512, 3)
    a = P.forward(cfg, w, ids)
    w["lm_head.weight"] = rng(19).normal(size=(512, 160))       # ignored when tied
    assert np.array_equal(P.forward(cfg, w, ids), a)
    untied = dict(cfg, tie_word_embeddings=False)
    assert not np.allclose(P.forward(untied, w, ids), a)


def test_window_config_changes_only_what_lies_beyond_the_window(weights):
    cfg = tc.TINY_C
    ids = tc.random_ids(60, 300, 4)
    with_window = P.forward(cfg, weights["C"], ids)
    without = P.forward(dict(cfg, sliding_window=None), weights["C"], ids)
    assert np.allclose(with_window[:24], without[:24], atol=1e-12)      # the first 24 positions see everything either way
    assert not np.allclose(with_window[30:], without[30:], atol=1e-6)


def test_llama3_band_interpolates_the_frequency_not_the_divisor():
    """Inside the band the scaled frequency f / divisor is a straight line in f between f / factor at the band's low end
    and f at its high end (rust/checkpoint/src/plan.rs:1495-1499), so 1 / divisor is a straight line in the wavelength's
    inverse: a lane in the middle of the band has divisor 1 / ((1/factor + 1) / 2), not (factor + 1) / 2; the ends join
    the regions outside without a step."""
    factor, low, high, original = 8.0, 1.0, 4.0, 8192.0
    dims = 64
    d = P.llama3_divisors(dims, 500000.0, factor, low, high, original).astype(np.float64)
    lanes = np.arange(dims // 2)
    wavelength = 2 * math.pi * 500000.0 ** (2 * lanes / dims)
    inside = (wavelength >= original / high) & (wavelength <= original / low)
    assert inside.sum() >= 3
    smooth = (original / wavelength[inside] - low) / (high - low)
    assert np.allclose(1.0 / d[inside], (1 - smooth) / factor + smooth, rtol=1e-6)
    assert not np.allclose(d[inside], (1 - smooth) * factor + smooth, rtol=1e-2)
    # a wavelength exactly in the middle of the band (theta chosen so that lane 1 of 4 dims has it)
    middle = original / ((low + high) / 2)
    theta = (middle / (2 * math.pi)) ** 2                  # lane 1: wavelength 2 pi theta^(2/4)
    assert abs(P.llama3_divisors(4, theta, factor, low, high, original)[1] - 1.0 / ((1.0 / factor + 1.0) / 2.0)) < 1e-5
    # the band's ends
    for edge, want in ((original / high, 1.0), (original / low, factor)):
        theta = (edge * (1 + 1e-9) / (2 * math.pi)) ** 2
        assert abs(P.llama3_divisors(4, theta, factor, low, high, original)[1] - want) < 1e-5


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_one_token_reduces_to_library_routines(weights, name):
    """A sequence of one token attends to itself alone: the attention weights are 1 whatever q, k and the rotation are,
    and the model is norms, matrix products, an activation and sums.  Written out with the library's routines in the
    order of a pre-norm layer (the branch reads the normed stream and adds to the stream that was not normed; the last
    norm comes before the head), it gives the plain implementation's logits; with a norm in another place it does not."""
    cfg = tc.CONFIGS[name]
    w = {k: torch.tensor(v) for k, v in weights[name].items()}
    sizes = P.read_sizes(cfg)
    group = sizes["heads"] // sizes["kv_heads"]
    d = sizes["head_dim"]

    def library(token, prenorm=True):
        x = w["model.embed_tokens.weight"][token]
        for i in range(sizes["layers"]):
            p = f"model.layers.{i}"
            h = F.rms_norm(x, x.shape, w[f"{p}.input_layernorm.weight"], eps=sizes["eps"])
            v = F.linear(h if prenorm else x, w[f"{p}.self_attn.v_proj.weight"], w.get(f"{p}.self_attn.v_proj.bias"))
            per_head = v.reshape(sizes["kv_heads"], d).repeat_interleave(group, dim=0).reshape(-1)
            x = x + F.linear(per_head, w[f"{p}.self_attn.o_proj.weight"], w.get(f"{p}.self_attn.o_proj.bias"))
            h = F.rms_norm(x, x.shape, w[f"{p}.post_attention_layernorm.weight"], eps=sizes["eps"])
            act = F.silu(F.linear(h, w[f"{p}.mlp.gate_proj.weight"], w.get(f"{p}.mlp.gate_proj.bias"))) * \
                F.linear(h, w[f"{p}.mlp.up_proj.weight"], w.get(f"{p}.mlp.up_proj.bias"))
            x = x + F.linear(act, w[f"{p}.mlp.down_proj.weight"], w.get(f"{p}.mlp.down_proj.bias"))
        x = F.rms_norm(x, x.shape, w["model.norm.weight"], eps=sizes["eps"])
        head = w["model.embed_tokens.weight"] if sizes["tied"] else w["lm_head.weight"]
        return F.linear(x, head).numpy()

    for token in (0, 7, cfg["vocab_size"] - 1):
        got = P.forward(cfg, weights[name], [token], first_position=5)[0]
        assert np.allclose(got, library(token), rtol=1e-9, atol=1e-12)
        assert not np.allclose(got, library(token, prenorm=False), rtol=1e-3)


def test_without_branches_the_model_is_norm_and_head(weights):
    """Output and down projections of zero: every layer adds nothing and the logits are head(norm(embedding)), for
    every token of a sequence."""
    cfg = tc.TINY_A
    w = dict(weights["A"])
    for i in range(cfg["num_hidden_layers"]):
        for n in ("self_attn.o_proj", "mlp.down_proj"):
            w[f"model.layers.{i}.{n}.weight"] = np.zeros_like(w[f"model.layers.{i}.{n}.weight"])
    ids = tc.random_ids(9, 256, 8)
    e = torch.tensor(w["model.embed_tokens.weight"])[ids]
    want = F.linear(F.rms_norm(e, (64,), torch.tensor(w["model.norm.weight"]), eps=1e-5), torch.tensor(w["lm_head.weight"]))
    assert np.allclose(P.forward(cfg, w, ids), want.numpy(), rtol=1e-10)


# ---- sampling --------------------------------------------------------------------------------
def test_philox_known_answers():
    """rust/engine/src/sampling.rs:1018-1030 (Random123's vectors for philox4x32, 10 rounds)."""
    assert P.philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert P.philox4x32_10([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    pi_digits = P.philox4x32_10([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0])
    assert pi_digits == [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_philox_uniforms():
    """rust/engine/src/sampling.rs:1032-1046."""
    us = np.array([P.philox_uniform(42, i, 0) for i in range(4000)])
    assert us.min() > 0.0 and us.max() < 1.0
    assert np.all(np.abs(np.histogram(us, bins=8, range=(0, 1))[0] - 500) < 100)
    assert P.philox_uniform(1, 0, 0) != P.philox_uniform(2, 0, 0) and P.philox_uniform(1, 0, 0) != P.philox_uniform(1, 0, 1)
    assert P.philox_uniform(7, 3, 9) == P.philox_uniform(7, 3, 9)
    many = P.philox_uniform_many((5 << 40) + 77, (3 << 33) + 9, np.array([0, 1, 2, 70000, 0xFFFFFFFF]))
    assert many.dtype == np.float32
    assert many.tolist() == [P.philox_uniform((5 << 40) + 77, (3 << 33) + 9, i) for i in (0, 1, 2, 70000, 0xFFFFFFFF)]


def test_greedy_takes_the_first_maximum():
    """rust/engine/src/sampling.rs:763-766."""
    assert P.greedy([0.1, 0.9, 0.9, -1.0]) == 1
    assert P.device_sample([0.1, 0.9, 0.9, float("nan")], 0.0, 0, 1.0, 1, 0) == 1


def test_filters():
    """The reference's vectors (rust/engine/src/sampling.rs:1061-1075): logits [3, 2, 1, 0, -1] at
    temperature 1: top_k 3 keeps ids 0, 1, 2; top_p 0.7 keeps two tokens."""
    logits = [3.0, 2.0, 1.0, 0.0, -1.0]
    alive = lambda **kw: np.flatnonzero(np.isfinite(P.device_survivors(logits, 1.0, kw.get("top_k", 0), kw.get("top_p", 1.0)))).tolist()
    assert alive(top_k=3) == [0, 1, 2] and alive(top_p=0.7) == [0, 1] and alive() == [0, 1, 2, 3, 4]
    assert alive(top_k=3, top_p=0.7) == [0, 1]
    assert np.flatnonzero(np.isfinite(P.device_survivors([1.0, 5.0, 5.0, 0.0], 1.0, 1, 1.0))).tolist() == [1, 2]   # ties are kept
    # a dominant token always survives top-p (sampling.rs:809-823)
    assert np.flatnonzero(np.isfinite(P.device_survivors([0.0, 20.0, 1.0], 1.0, 0, 0.1))).tolist() == [1]


def test_min_p_and_the_order_of_the_filters():
    """The reference's vectors: logits [3, 2, 1, 0, -1] at temperature 1 with min_p 0.3 keep two tokens
    (rust/engine/src/sampling.rs:1069-1070: e^-1 = 0.37 stays, e^-2 = 0.14 goes); [5, 3, 0] with min_p 0.5 leave
    token 0 alone (:842-856).  top-k comes first, min-p next, top-p last, each over what the one before left."""
    alive = lambda logits, **kw: np.flatnonzero(np.isfinite(P.device_survivors(
        logits, kw.get("t", 1.0), kw.get("top_k", 0), kw.get("top_p", 1.0), kw.get("min_p", 0.0)))).tolist()
    assert alive([3.0, 2.0, 1.0, 0.0, -1.0], min_p=0.3) == [0, 1]
    assert alive([5.0, 3.0, 0.0], min_p=0.5) == [0]
    assert all(P.device_sample([5.0, 3.0, 0.0], 1.0, 0, 1.0, 1, d, min_p=0.5) == 0 for d in range(50))
    # the weight is taken at the temperature: at T = 2, e^(-2/2) = 0.37 stays where at T = 1 e^-2 went
    assert alive([3.0, 2.0, 1.0, 0.0, -1.0], min_p=0.3, t=2.0) == [0, 1, 2]
    # top-p over what min-p left: of [3, 2] (weights 1, 0.37) top_p 0.7 needs only the first; without min-p, of all five, it needs two
    assert alive([3.0, 2.0, 1.0, 0.0, -1.0], min_p=0.3, top_p=0.7) == [0]
    assert alive([3.0, 2.0, 1.0, 0.0, -1.0], top_p=0.7) == [0, 1]
    assert alive([3.0, 3.0, 2.9, 0.0], top_k=1, min_p=0.5) == [0, 1]        # ties of top-k stay, min-p has nothing to add


def test_penalties_and_controls():
    """The reference's vectors: repetition penalty 2 turns logits [4, 6, 1] with token 1 in the history into a win for
    token 0 (rust/engine/src/sampling.rs:776-791); frequency 1.0 and presence 0.5 over the last 2 tokens of [0, 1, 1]
    turn [5, 5] into [5, 2.5] (:857-868).  A negative logit is multiplied, not divided; a token counts once for the
    repetition penalty however often it occurs; biases come last; min_tokens blocks end and stop ids until reached."""
    assert P.greedy(P.apply_penalties([4.0, 6.0, 1.0], [1], repetition_penalty=2.0)) == 0
    assert P.apply_penalties([5.0, 5.0], [0, 1, 1], frequency_penalty=1.0, presence_penalty=0.5, repeat_last_n=2).tolist() == [5.0, 2.5]
    assert P.apply_penalties([5.0, 5.0], [0, 1, 1], frequency_penalty=1.0, presence_penalty=0.5).tolist() == [3.5, 2.5]
    assert P.apply_penalties([-2.0, 2.0, 1.0], [0, 0, 1], repetition_penalty=2.0).tolist() == [-4.0, 1.0, 1.0]
    assert P.apply_penalties([1.0, 1.0], [0], repetition_penalty=1.000001).tolist() == [1.0, 1.0]      # as good as 1: off
    assert P.apply_penalties([1.0, 1.0, 1.0], [7, -1, 1], presence_penalty=0.25, logit_bias=[(2, -3.0), (9, 1.0)]).tolist() == [1.0, 0.75, -2.0]
    assert P.apply_penalties([4.0], [0], repetition_penalty=2.0, logit_bias=[(0, 1.0)]).tolist() == [3.0]   # the bias after the penalty
    blocked = P.apply_generation_controls([1.0, 2.0, 3.0, 4.0], 3, 2, [3], [1])
    assert np.isneginf(blocked[[1, 3]]).all() and blocked[[0, 2]].tolist() == [1.0, 3.0]
    assert P.apply_generation_controls([1.0, 2.0, 3.0, 4.0], 3, 3, [3], [1]).tolist() == [1.0, 2.0, 3.0, 4.0]


def test_allow_list_and_bad_words():
    """rust/engine/src/sampling.rs:228-249.  An allow list of one token forces it (how rust/engine/src/beam_tests.rs:130
    scores a given continuation), one of all tokens changes nothing, ids outside the vocabulary are ignored; a bad
    word blocks its last token only behind its other tokens, a word of one token always, a word longer than the
    history never."""
    row = np.array([0.5, 3.0, -1.0, 2.0, 0.0], dtype=np.float32)
    forced = P.apply_generation_controls(row, 0, 0, (), (), allowed_token_ids=(2, 9))
    assert P.greedy(forced) == 2 and np.isinf(forced[[0, 1, 3, 4]]).all() and forced[2] == row[2]
    assert np.array_equal(P.apply_generation_controls(row, 0, 0, (), (), allowed_token_ids=range(5)), row)
    words = ((1,), (4, 3), (0, 4, 0), (2, 2, 2, 2, 2, 2, 3))
    assert np.array_equal(np.isinf(P.apply_generation_controls(row, 0, 0, (), (), (), words, history=[0, 4])), [True, True, False, True, False])
    assert np.array_equal(np.isinf(P.apply_generation_controls(row, 0, 0, (), (), (), words, history=[4, 0])), [False, True, False, False, False])
    assert np.array_equal(np.isinf(P.apply_generation_controls(row, 0, 0, (), (), (), words, history=[])), [False, True, False, False, False])
    # all of them together with min_tokens: what each blocks adds up
    out = P.apply_generation_controls(row, 2, 1, (3,), (0,), (0, 2, 3, 4), ((2, 4),), history=[2])
    assert np.array_equal(np.isinf(out), [True, True, False, True, True])


def test_raw_logprobs():
    """rust/engine/src/sampling.rs:970-978: stable around the largest value, ties in token order, no distribution for bad rows."""
    logprob, top = P.raw_logprobs([1000.0, 1000.0, 999.0], 2, 2)
    assert [i for i, _ in top] == [0, 1]
    assert abs(logprob - (-1.0 - math.log(2.0 + math.exp(-1.0)))) < 1e-12
    big = float(np.finfo(np.float32).max)
    assert abs(P.raw_logprobs([big, big], 0, 0)[0] + math.log(2.0)) < 1e-12
    assert P.raw_logprobs([float("nan")], 0, 1) is None and P.raw_logprobs([-np.inf], 0, 1) is None
    # it is the library's log-softmax, and at most 20 alternatives come back
    rng = np.random.default_rng(5)
    w = rng.normal(size=300).astype(np.float32) * 4
    logprob, top = P.raw_logprobs(w, 17, 50)
    want = torch.log_softmax(torch.from_numpy(w).double(), 0)
    assert abs(logprob - float(want[17])) < 1e-12 and len(top) == 20
    assert [i for i, _ in top] == torch.argsort(want, descending=True, stable=True)[:20].tolist()


def test_processed_logprobs():
    """rust/engine/src/sampling.rs:1542-1556: the reference's own vector (only the survivors of top-k are listed, their
    probabilities add up to one, a token outside the support has probability zero, greedy is a point mass), and the
    softmax of logits / T over what the filters leave against the library's."""
    logits = [3.0, 2.0, 1.0, 0.0, -1.0]
    chosen, top = P.processed_logprobs(logits, 1, 5, 1.0, top_k=3)
    assert [i for i, _ in top] == [0, 1, 2] and abs(sum(math.exp(v) for _, v in top) - 1.0) < 1e-6
    assert abs(chosen - top[1][1]) < 1e-12
    assert P.processed_logprobs(logits, 4, 5, 1.0, top_k=3)[0] == -math.inf
    assert P.processed_logprobs(logits, 0, 3, 0.0) == (0.0, [(0, 0.0)])
    assert P.processed_logprobs(logits, 2, 3, 0.0)[0] == -math.inf
    assert P.processed_logprobs([-np.inf, float("nan")], 0, 1, 1.0) is None
    rng = np.random.default_rng(8)
    w = rng.normal(size=200).astype(np.float32) * 3
    # no filter: log-softmax of w / T
    chosen, top = P.processed_logprobs(w, 17, 20, 0.7)
    want = torch.log_softmax(torch.from_numpy(w).double() / 0.7, 0)
    assert abs(chosen - float(want[17])) < 1e-5 and [i for i, _ in top] == torch.argsort(want, descending=True, stable=True)[:20].tolist()
    # top-k 6 and top-p 0.5: the renormalized head of that distribution; min-p drops what is 20 times lighter than the top
    order = torch.argsort(want, descending=True, stable=True).tolist()
    head = want[order[:6]].exp()
    kept = int(np.flatnonzero(np.cumsum((head / head.sum()).numpy()) >= 0.5)[0]) + 1
    chosen, top = P.processed_logprobs(w, order[0], 20, 0.7, top_k=6, top_p=0.5)
    assert [i for i, _ in top] == order[:kept] and abs(sum(math.exp(v) for _, v in top) - 1.0) < 1e-6
    assert abs(chosen - math.log(float(head[0] / head[:kept].sum()))) < 1e-5
    assert P.processed_logprobs(w, order[kept], 20, 0.7, top_k=6, top_p=0.5)[0] == -math.inf
    _, top = P.processed_logprobs(w, order[0], 20, 0.7, min_p=0.05)
    assert [i for i, _ in top] == [i for i in order if float(want[i] - want[order[0]]) >= math.log(0.05)][:20]


def test_draws_follow_the_distribution_and_depend_on_seed_and_draw_only():
    logits = np.array([2.0, 1.0, 0.0, -1.0], dtype=np.float32)
    p = np.exp(logits / 0.8)
    p /= p.sum()
    counts = np.bincount([P.device_sample(logits, 0.8, 0, 1.0, 5, d) for d in range(3000)], minlength=4) / 3000
    assert np.all(np.abs(counts - p) < 0.03)
    assert P.device_sample(logits, 0.8, 0, 1.0, 5, 17) == P.device_sample(logits, 0.8, 0, 1.0, 5, 17)
    assert len({P.device_sample(logits, 1.5, 0, 1.0, s, 0) for s in range(40)}) > 1


def test_the_smoke_run_carries_the_same_plain_model(weights):
    """__graft_entry__.smoke() compares the engine with a plain model of its own, so that it runs from that file and the
    package alone; here that one is held against this folder's."""
    import __graft_entry__ as entry
    cfg = entry.SMOKE_CONFIG
    assert cfg == {k: v for k, v in tc.TINY_A.items()}
    ids = tc.random_ids(23, cfg["vocab_size"], 5)
    assert np.allclose(entry.plain_logits(cfg, weights["A"], ids), P.forward(cfg, weights["A"], ids), rtol=0, atol=1e-12)
