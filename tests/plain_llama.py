"""A plain, slow Llama: whole sequences, no cache, float64, one function per part.

Written from the reference's formulas (file:line cited per function, paths relative to the
reference's root); it shares no code with `fllm_amd`.  Weights come in as a dict of float64
NumPy arrays under the checkpoint's tensor names, the configuration as the config.json dict.
"""
import math

import numpy as np


# ---------------------------------------------------------------------------------------------
# configuration, read straight from config.json keys (rust/checkpoint/src/plan.rs:1066-1111 sizes,
# :1222-1236 eps, :1239-1287 window, :92-121 and :1323-1338 rotary base, :1478-1505 llama3)
# ---------------------------------------------------------------------------------------------
def read_sizes(cfg):
    hidden = cfg["hidden_size"]
    heads = cfg["num_attention_heads"]
    out = {
        "hidden": hidden,
        "layers": cfg["num_hidden_layers"],
        "heads": heads,
        "kv_heads": cfg.get("num_key_value_heads", heads),
        "head_dim": cfg.get("head_dim", hidden // heads),
        "inter": cfg["intermediate_size"],
        "vocab": cfg.get("vocab_size", 32000),
        "eps": cfg.get("rms_norm_eps", 1e-6),
        "tied": bool(cfg.get("tie_word_embeddings", False)),
    }
    scaling = cfg.get("rope_scaling") or {}
    params = cfg.get("rope_parameters") or {}
    if params:
        scaling = params
    out["theta"] = float(scaling.get("rope_theta", cfg.get("rope_theta", 10000.0)))
    out["rope_kind"] = str(scaling.get("rope_type", scaling.get("type", "default"))).lower()
    out["rope_scaling"] = scaling
    out["context"] = out["model_context"] = cfg.get("max_position_embeddings", 40960)
    if out["rope_kind"] == "dynamic" and "alpha" in scaling:
        # rust/checkpoint/src/plan.rs:1339-1343: the base grows, nothing else of the scaling stays (:1376)
        d = float(out["head_dim"])
        out["theta"] *= float(scaling["alpha"]) ** (d / (d - 2.0))
        out["rope_kind"] = "default"
    partial = cfg.get("partial_rotary_factor", 1.0)
    out["rope_dims"] = int(round(out["head_dim"] * partial))
    window = cfg.get("sliding_window") or 0
    layers = out["layers"]
    if window > 0 and cfg.get("use_sliding_window") is not False:
        types = cfg.get("layer_types")
        if isinstance(types, list) and len(types) == layers:
            out["windows"] = [window if t == "sliding_attention" else None for t in types]
        else:
            out["windows"] = [window] * layers
    else:
        out["windows"] = [None] * layers
    return out


# ---------------------------------------------------------------------------------------------
# parts
# ---------------------------------------------------------------------------------------------
def rms_norm(x, weight, eps):
    """rust/engine/src/rust_decoder.rs:1481-1490: inv = 1/sqrt(sum(x^2)/n + eps); x *= inv * w."""
    x = np.asarray(x, dtype=np.float64)
    inv = 1.0 / np.sqrt((x * x).sum(axis=-1, keepdims=True) / x.shape[-1] + eps)
    return x * (inv * np.asarray(weight, dtype=np.float64))


def llama3_divisors(dims, theta, factor, low, high, original):
    """rust/checkpoint/src/plan.rs:1478-1505: float64 per-lane divisors, cast to float32."""
    out = []
    low_wavelength = original / low
    high_wavelength = original / high
    for i in range(dims // 2):
        frequency = 1.0 / theta ** ((2 * i) / dims)
        wavelength = 2.0 * math.pi / frequency
        if wavelength < high_wavelength:
            scale = 1.0
        elif wavelength > low_wavelength:
            scale = factor
        else:
            smooth = (original / wavelength - low) / (high - low)
            scale = 1.0 / ((1.0 - smooth) / factor + smooth)
        out.append(np.float32(scale))
    return np.array(out, dtype=np.float32)


def yarn_values(scaling, cfg_original=None):
    """What the engine's YaRN tables are built from, out of the keys of config.json
    (rust/checkpoint/src/plan.rs:1433-1477 writes them as float32 metadata, rust/engine/src/config.rs:1558-1569 reads
    them with these defaults): the checkpoint's `attention_factor` (or mscale quotient) h replaces the built-in
    magnitude 1 + 0.1 ln(factor), so the engine's factor is h / (1 + 0.1 ln(factor))."""
    factor = float(scaling["factor"])
    magnitude = lambda m: 0.1 * m * math.log(factor) + 1.0
    h = scaling.get("attention_factor")
    if h is None and "mscale" in scaling and "mscale_all_dim" in scaling:
        h = magnitude(float(scaling["mscale"])) / magnitude(float(scaling["mscale_all_dim"]))
    return {
        "factor": np.float32(factor),
        "original": int(scaling.get("original_max_position_embeddings", cfg_original)),
        "extrapolation": np.float32(scaling.get("extrapolation_factor", 1.0)),
        "attention": np.float32(1.0 if h is None else float(h) / magnitude(1.0)),
        "beta_fast": np.float32(scaling.get("beta_fast", 32.0)),
        "beta_slow": np.float32(scaling.get("beta_slow", 1.0)),
        "truncate": scaling.get("truncate") is not False,
    }


def yarn_tables(positions, inverse, dims, base, y):
    """rust/engine/src/rope.rs:70-110 with :15-23, all in float32 up to the phase: a lane's angle is a mix of the
    plain angle (position * inverse) and the interpolated one (that divided by the factor); the lanes below the
    correction dimension of `beta_fast` keep the plain angle, those above that of `beta_slow` the interpolated
    one, a straight ramp between; cos and sin are multiplied by attention * (1 + 0.1 ln(factor))."""
    f = np.float32
    two_pi = f(2.0) * f(math.pi)

    def correction_dim(rotations):
        return f(f(dims) * np.log(f(f(y["original"]) / f(rotations * two_pi))) / f(f(2.0) * np.log(f(base))))

    low, high = correction_dim(y["beta_fast"]), correction_dim(y["beta_slow"])
    if y["truncate"]:
        low, high = np.floor(low), np.ceil(high)
    low, high = max(low, f(0.0)), min(high, f(dims - 1))
    scale = f(1.0) / y["factor"]
    lanes = np.arange(len(inverse), dtype=np.float32)
    ramp = f(1.0) - np.clip((lanes - low) / max(f(high - low), f(0.001)), f(0.0), f(1.0)).astype(np.float32)
    pos = np.asarray(positions, dtype=np.float32)
    extrapolated = (pos[:, None] * inverse[None, :]).astype(np.float32)
    interpolated = (scale * extrapolated).astype(np.float32)
    if y["extrapolation"] != 0.0:
        mix = (ramp * y["extrapolation"]).astype(np.float32)[None, :]
        theta = (interpolated * (f(1.0) - mix) + extrapolated * mix).astype(np.float32)
        magnitude = f(y["attention"] * f(f(1.0) + f(0.1) * np.log(f(f(1.0) / scale))))
    else:
        theta, magnitude = interpolated, y["attention"]
    phase = theta.astype(np.float64)
    cos = (np.cos(phase).astype(np.float32) * magnitude).astype(np.float32)
    sin = (np.sin(phase).astype(np.float32) * magnitude).astype(np.float32)
    return cos.astype(np.float64), sin.astype(np.float64)


def longrope_values(scaling, dims, context):
    """rust/checkpoint/src/plan.rs:1507-1548: the two lists of dims/2 factors, the original context (the model's
    own context when the key is missing) and the factor on cos and sin: `attention_factor`, else
    sqrt(1 + ln(context / original) / ln(original)) when the context is longer than the original one, else 1."""
    short = np.array(scaling["short_factor"], dtype=np.float32)
    long = np.array(scaling["long_factor"], dtype=np.float32)
    assert len(short) == len(long) == dims // 2
    original = int(scaling.get("original_max_position_embeddings", context))
    ratio = context / original
    attention = scaling.get("attention_factor")
    if attention is None:
        attention = math.sqrt(1.0 + math.log(ratio) / math.log(original)) if ratio > 1.0 else 1.0
    return short, long, original, np.float32(attention)


def rope_tables(positions, dims, theta, kind="default", scaling=None, context=None, model_context=None):
    """rust/engine/src/rope.rs:38-68: inverse frequencies in float32 (divided by the per-lane
    divisors when there are any), phase = position * inverse in float32 (`linear` scaling divides
    the position, :53-62), cos and sin in float64.  `yarn`: see yarn_tables.  `longrope` (:30-36, :58-66): the
    frequencies are divided by the long factors when the engine's tables reach beyond the original context
    (`context` positions; the model's own context, `model_context`, when left out), by the short ones otherwise,
    and cos and sin are multiplied by the attention factor in float32.  Returns float64 [len(positions), dims/2]."""
    scaling = scaling or {}
    half = dims // 2
    lanes = np.arange(half, dtype=np.float32)
    exponent = (lanes * np.float32(2.0)) / np.float32(dims)
    # `base.powf(exponent)` on float32 operands: the correctly rounded float32 power
    power = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)
    inverse = (np.float32(1.0) / power).astype(np.float32)
    scale = np.float32(1.0)
    if kind == "llama3":
        inverse = (inverse / llama3_divisors(dims, theta, float(scaling["factor"]),
                                             float(scaling.get("low_freq_factor", 1.0)),
                                             float(scaling.get("high_freq_factor", 4.0)),
                                             float(scaling["original_max_position_embeddings"]))).astype(np.float32)
    elif kind == "linear":
        scale = np.float32(1.0) / np.float32(scaling["factor"])
    elif kind == "yarn":
        return yarn_tables(positions, inverse, dims, np.float32(theta), yarn_values(scaling))
    elif kind in ("longrope", "su"):
        model_context = model_context or context or 40960
        short, long, original, magnitude = longrope_values(scaling, dims, model_context)
        inverse = (inverse / (long if (context or model_context) > original else short)).astype(np.float32)
    elif kind != "default":
        raise ValueError(kind)
    pos = np.asarray(positions, dtype=np.float32) * scale
    phase = (pos[:, None] * inverse[None, :]).astype(np.float32).astype(np.float64)
    if kind in ("longrope", "su"):
        cos = (np.cos(phase).astype(np.float32) * magnitude).astype(np.float32)
        sin = (np.sin(phase).astype(np.float32) * magnitude).astype(np.float32)
        return cos.astype(np.float64), sin.astype(np.float64)
    return np.cos(phase), np.sin(phase)


def apply_rope(x, cos, sin, dims, interleaved=False):
    """rust/engine/src/rust_decoder.rs:1655-1683: rotate lane pairs of the first `dims` values of
    every head: (a, b) <- (a cos - b sin, b cos + a sin).  The reference pairs (2l, 2l+1) on
    weights whose q/k rows it permuted at import (rust/checkpoint/src/convert.rs:2713-2745); on the
    checkpoint's own row order that is the pairing (l, l + dims/2), used here unless `interleaved`.
    x: [tokens, heads, head_dim]; cos, sin: [tokens, dims/2]."""
    x = np.array(x, dtype=np.float64, copy=True)
    half = dims // 2
    if interleaved:
        ia, ib = np.arange(half) * 2, np.arange(half) * 2 + 1
    else:
        ia, ib = np.arange(half), np.arange(half) + half
    a, b = x[:, :, ia].copy(), x[:, :, ib].copy()
    c, s = cos[:, None, :], sin[:, None, :]
    x[:, :, ia] = a * c - b * s
    x[:, :, ib] = b * c + a * s
    return x


def attention(q, k, v, scale, window=None):
    """rust/engine/src/rust_decoder.rs:6065-6166: row r (position r, length n = r + 1) sees keys
    start..n with start = n - window (0 without a window, :6090-6093); head h uses key/value head
    h / (heads / kv_heads) (:6121); s = (q . k) * scale; softmax over the visible keys; weights
    are divided by their sum before they multiply v (:6156-6161).
    q: [T, heads, d]; k, v: [T, kv_heads, d] -> [T, heads, d]."""
    T, heads, d = q.shape
    kv_heads = k.shape[1]
    group = heads // kv_heads
    out = np.zeros((T, heads, v.shape[2]), dtype=np.float64)
    for r in range(T):
        n = r + 1
        start = 0 if window is None else max(0, n - window)
        for h in range(heads):
            kh = h // group
            scores = (k[start:n, kh, :] @ q[r, h, :]) * scale
            e = np.exp(scores - scores.max())
            w = e / e.sum()
            out[r, h, :] = w @ v[start:n, kh, :]
    return out


def silu(x):
    """rust/engine/src/rust_decoder.rs:1645: x / (1 + exp(-x))."""
    return x / (1.0 + np.exp(-x))


def linear(x, weight, bias=None):
    """rust/engine/src/compute.rs:292-308: y[b][r] = sum_k x[b][k] W[r][k] (+ bias[r])."""
    y = x @ np.asarray(weight, dtype=np.float64).T
    if bias is not None:
        y = y + np.asarray(bias, dtype=np.float64)
    return y


def gated_mlp(x, gate, up, down, gate_bias=None, up_bias=None, down_bias=None):
    """rust/engine/src/rust_decoder.rs:8328-8352: down(silu(gate x) * (up x))."""
    return linear(silu(linear(x, gate, gate_bias)) * linear(x, up, up_bias), down, down_bias)


def attention_layer(x, weights, prefix, sizes, layer, positions):
    """rust/engine/src/rust_decoder.rs:8827-8835 (projections), :8895-8898 (rotary on q and k),
    :8976-9001 (attention), :9025 (output projection)."""
    T = x.shape[0]
    heads, kv_heads, d = sizes["heads"], sizes["kv_heads"], sizes["head_dim"]
    g = lambda n: weights.get(f"{prefix}.self_attn.{n}")
    q = linear(x, g("q_proj.weight"), g("q_proj.bias")).reshape(T, heads, d)
    k = linear(x, g("k_proj.weight"), g("k_proj.bias")).reshape(T, kv_heads, d)
    v = linear(x, g("v_proj.weight"), g("v_proj.bias")).reshape(T, kv_heads, d)
    cos, sin = rope_tables(positions, sizes["rope_dims"], sizes["theta"], sizes["rope_kind"], sizes["rope_scaling"],
                           sizes.get("context"), sizes.get("model_context"))
    q = apply_rope(q, cos, sin, sizes["rope_dims"])
    k = apply_rope(k, cos, sin, sizes["rope_dims"])
    o = attention(q, k, v, 1.0 / math.sqrt(d), sizes["windows"][layer])
    return linear(o.reshape(T, heads * d), g("o_proj.weight"), g("o_proj.bias"))


def forward(cfg, weights, token_ids, first_position=0, context=None):
    """Logits [T, vocab] of a whole sequence (rust/engine/src/rust_decoder.rs:8531-8701 and
    :8706-9117): embedding; per layer x += attention(norm(x)), x += mlp(norm(x)); final norm;
    head (the embedding table when `tie_word_embeddings`, rust_decoder.rs:2503-2507).  `context`: the positions the
    engine is set up for (rust/engine/src/model.rs:307), the model's own context when left out; only `longrope`
    looks at it."""
    sizes = read_sizes(cfg)
    if context is not None:
        sizes["context"] = context
    ids = np.asarray(token_ids, dtype=np.int64)
    positions = np.arange(first_position, first_position + len(ids))
    x = np.asarray(weights["model.embed_tokens.weight"], dtype=np.float64)[ids]
    for i in range(sizes["layers"]):
        p = f"model.layers.{i}"
        h = rms_norm(x, weights[f"{p}.input_layernorm.weight"], sizes["eps"])
        x = x + attention_layer(h, weights, p, sizes, i, positions)
        h = rms_norm(x, weights[f"{p}.post_attention_layernorm.weight"], sizes["eps"])
        x = x + gated_mlp(h, weights[f"{p}.mlp.gate_proj.weight"], weights[f"{p}.mlp.up_proj.weight"],
                          weights[f"{p}.mlp.down_proj.weight"], weights.get(f"{p}.mlp.gate_proj.bias"),
                          weights.get(f"{p}.mlp.up_proj.bias"), weights.get(f"{p}.mlp.down_proj.bias"))
    x = rms_norm(x, weights["model.norm.weight"], sizes["eps"])
    head = weights["model.embed_tokens.weight"] if sizes["tied"] else weights["lm_head.weight"]
    return linear(x, head)


# ---------------------------------------------------------------------------------------------
# sampling
# ---------------------------------------------------------------------------------------------
def greedy(logits):
    """rust/engine/src/sampling.rs:531-552: the first position of the largest value."""
    logits = np.asarray(logits)
    return int(np.flatnonzero(logits == logits.max())[0])


_M0, _M1, _W0, _W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85


def philox4x32_10(ctr, key):
    """rust/engine/src/sampling.rs:155-172."""
    c = [int(v) & 0xFFFFFFFF for v in ctr]
    k = [int(v) & 0xFFFFFFFF for v in key]
    for _ in range(10):
        p0 = _M0 * c[0]
        p1 = _M1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, p1 & 0xFFFFFFFF,
             ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF, p0 & 0xFFFFFFFF]
        k = [(k[0] + _W0) & 0xFFFFFFFF, (k[1] + _W1) & 0xFFFFFFFF]
    return c


def philox_uniform(seed, draw, index):
    """rust/engine/src/sampling.rs:174-183: ((w >> 8) + 0.5) / 2^24 in float32, in (0, 1)."""
    w = philox4x32_10([index, 0, draw & 0xFFFFFFFF, draw >> 32], [seed & 0xFFFFFFFF, seed >> 32])[0]
    return np.float32((np.float32(w >> 8) + np.float32(0.5)) / np.float32(16777216.0))


def philox_uniform_many(seed, draw, indices):
    """philox_uniform for an array of indices at once (the same arithmetic on uint64 arrays)."""
    mask = np.uint64(0xFFFFFFFF)
    c = [np.asarray(indices, dtype=np.uint64) & mask, np.zeros(len(indices), np.uint64),
         np.full(len(indices), draw & 0xFFFFFFFF, np.uint64), np.full(len(indices), draw >> 32, np.uint64)]
    k0, k1 = seed & 0xFFFFFFFF, seed >> 32
    for _ in range(10):
        p0 = np.uint64(_M0) * c[0]
        p1 = np.uint64(_M1) * c[2]
        c = [((p1 >> np.uint64(32)) ^ c[1] ^ np.uint64(k0)) & mask, p1 & mask,
             ((p0 >> np.uint64(32)) ^ c[3] ^ np.uint64(k1)) & mask, p0 & mask]
        k0, k1 = (k0 + _W0) & 0xFFFFFFFF, (k1 + _W1) & 0xFFFFFFFF
    w = (c[0] >> np.uint64(8)).astype(np.float32)
    return ((w + np.float32(0.5)) / np.float32(16777216.0)).astype(np.float32)


def apply_generation_controls(logits, min_tokens, generated, eos_ids, stop_token_ids, allowed_token_ids=(), bad_word_ids=(),
                              history=()):
    """rust/engine/src/sampling.rs:220-250: while fewer than `min_tokens` tokens were generated, neither an
    end-of-sequence id nor a stop id can be chosen; with an allow list, nothing outside it; the last token of a bad
    word not when the word's other tokens are the end of `history` (prompt and generated tokens).  Returns a float32 copy."""
    out = np.asarray(logits, dtype=np.float32).copy()
    if generated < min_tokens:
        for t in list(eos_ids) + list(stop_token_ids):
            if 0 <= t < len(out):
                out[t] = -np.inf
    if len(allowed_token_ids):
        keep = np.zeros(len(out), dtype=bool)
        keep[[t for t in allowed_token_ids if 0 <= t < len(out)]] = True
        out[~keep] = -np.inf
    history = list(history)
    for word in bad_word_ids:
        if not len(word):
            continue
        before, last = list(word[:-1]), word[-1]
        if len(history) >= len(before) and history[len(history) - len(before):] == before and 0 <= last < len(out):
            out[last] = -np.inf
    return out


def raw_logprobs(logits, token, top_n):
    """rust/engine/src/sampling.rs:937-965: log-softmax of the float32 logits as they are, in float64 around the
    largest value: (log-probability of `token`, the min(top_n, 20) likeliest as (id, log-probability), the lower id
    first among equals).  A NaN or +inf anywhere, or no finite value at all, is an error there; here it is None."""
    w = np.asarray(logits, dtype=np.float32).astype(np.float64)
    if not 0 <= token < len(w) or np.isnan(w).any() or (w == np.inf).any() or not np.isfinite(w.max()):
        return None
    shifted = w - w.max()
    logp = shifted - math.log(np.exp(shifted).sum())
    order = sorted(range(len(w)), key=lambda i: (-logp[i], i))[:min(top_n, 20)]
    return float(logp[token]), [(i, float(logp[i])) for i in order]


def processed_logprobs(logits, token, top_n, temperature, top_k=0, top_p=1.0, min_p=0.0):
    """rust/engine/src/sampling.rs:365-381 and :928-935 (`logprobs_mode: processed_logprobs`): the log-probabilities of
    the distribution a token is drawn from.  A greedy request (temperature <= 1e-5) is a point mass on the first largest
    logit; otherwise the softmax of logits / T over the tokens the sampler still draws from (`device_survivors`, with its
    ties kept).  Returns (log-probability of `token`, -inf outside the support; the min(top_n, 20) likeliest of the
    tokens that are left as (id, log-probability), the lower id first among equals), or None without a finite logit."""
    w = np.asarray(logits, dtype=np.float32)
    finite = np.where(np.isfinite(w), w, -np.inf)
    if not np.isfinite(finite).any():
        return None
    if temperature <= 1e-5:
        first = greedy(finite)
        return (0.0 if token == first else -math.inf), [(first, 0.0)][:min(top_n, 20)]
    left = device_survivors(logits, temperature, top_k, top_p, min_p)
    alive = np.isfinite(left)
    inv_t = np.float32(1.0 / float(temperature))
    scaled = ((finite - finite.max()) * inv_t).astype(np.float32).astype(np.float64)
    log_mass = math.log(np.exp(scaled[alive]).sum())
    logp = np.where(alive, scaled - log_mass, -np.inf)
    order = sorted(np.flatnonzero(alive).tolist(), key=lambda i: (-logp[i], i))[:min(top_n, 20)]
    return float(logp[token]), [(i, float(logp[i])) for i in order]


def apply_penalties(logits, history, repetition_penalty=1.0, presence_penalty=0.0, frequency_penalty=0.0, repeat_last_n=-1,
                    logit_bias=()):
    """rust/engine/src/sampling.rs:252-274 and :579-598: over the last `repeat_last_n` tokens of the history (all of
    them when negative): every distinct token's logit is divided by the repetition penalty when positive and multiplied
    by it otherwise (once a token, and only if the penalty differs from 1 by 1e-5 or more); then presence +
    frequency * count is taken off; then the biases are added.  float32 arithmetic; returns a copy."""
    out = np.asarray(logits, dtype=np.float32).copy()
    tokens = list(history) if repeat_last_n < 0 else list(history)[max(0, len(history) - repeat_last_n):]
    tokens = [t for t in tokens if 0 <= t < len(out)]
    counts = {}
    for t in tokens:
        counts[t] = counts.get(t, 0) + 1
    rep = np.float32(repetition_penalty)
    if abs(float(rep) - 1.0) >= 1e-5:
        for t in counts:
            out[t] = out[t] / rep if out[t] > 0 else out[t] * rep
    for t, n in counts.items():
        out[t] = out[t] - (np.float32(presence_penalty) + np.float32(frequency_penalty) * np.float32(n))
    for t, b in logit_bias:
        if 0 <= t < len(out):
            out[t] = out[t] + np.float32(b)
    return out


def device_survivors(logits, temperature, top_k, top_p, min_p=0.0):
    """The tokens the reference's device sampler still draws from, as a float32 array of logits
    with -inf for the others (rust/engine/cuda/sampling.cu:253-330), with sorting in place of its
    bisections: non-finite logits never survive; top-k keeps everything not below the k-th
    largest value (ties kept); min-p (:294-300) then drops what weighs less than min_p times the
    largest weight, exp((v - max) / T) < min_p in float32; top-p keeps the largest values until their mass
    reaches top_p of the total of what is left (ties at the threshold kept)."""
    w = np.asarray(logits, dtype=np.float32).copy()
    w[~np.isfinite(w)] = -np.inf
    if not np.isfinite(w).any():
        return w
    m = w.max()
    inv_t = np.float32(1.0 / float(temperature))
    if 0 < top_k < len(w):
        kth = np.sort(w)[::-1][top_k - 1]
        w[w < kth] = -np.inf
    if min_p > 0.0:
        alive = np.isfinite(w)
        e = np.exp(((w[alive] - m) * inv_t).astype(np.float32)).astype(np.float32)
        keep = np.flatnonzero(alive)[e >= np.float32(min_p)]
        cut = np.full(len(w), -np.inf, dtype=np.float32)
        cut[keep] = w[keep]
        w = cut
    if 0.0 < top_p < 1.0:
        alive = np.isfinite(w)
        e = np.where(alive, np.exp(((w - m) * inv_t).astype(np.float32)).astype(np.float64), 0.0)
        target = float(np.float32(top_p)) * e.sum()
        values, inverse = np.unique(w[alive], return_inverse=True)           # distinct values, ascending
        per_value = np.bincount(inverse, weights=e[alive], minlength=len(values))
        mass = np.cumsum(per_value[::-1])                       # mass of {value >= v}, v descending
        threshold = values[::-1][np.flatnonzero(mass >= target)[0]]   # largest threshold that still reaches the target
        w[w < threshold] = -np.inf
    return w


def device_sample(logits, temperature, top_k, top_p, seed, draw, min_p=0.0):
    """rust/engine/cuda/sampling.cu:253-352: temperature <= 1e-5 is greedy; otherwise the token
    is the argmax over the survivors of (logit - max) / T - ln(-ln u_i),
    u_i = philox_uniform(seed, draw, i), lowest id on ties."""
    raw = np.asarray(logits, dtype=np.float32)
    finite = np.where(np.isfinite(raw), raw, -np.inf)
    if not np.isfinite(finite).any():
        return 0
    if temperature <= 1e-5:
        return greedy(finite)
    w = device_survivors(logits, temperature, top_k, top_p, min_p)
    m = finite.max()
    inv_t = np.float32(1.0 / float(temperature))
    alive = np.flatnonzero(np.isfinite(w))
    u = philox_uniform_many(seed, draw, alive)
    score = ((w[alive] - m) * inv_t).astype(np.float32) - np.log(-np.log(u, dtype=np.float32), dtype=np.float32)
    return int(alive[np.flatnonzero(score == score.max())[0]])
