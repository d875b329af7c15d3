"""Typed configuration of the Llama architecture, read from a checkpoint's config.json.

Keys, defaults and error texts follow the reference's checkpoint planner
(rust/checkpoint/src/plan.rs:879-1560 `from_config`): sizes at :1066-1111, activation at
:1129-1166, eps at :1222-1236, sliding window at :1239-1287, rotary parameters at :92-121 and
:1323-1548.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .files import read_config_json
from .spec import ConfigError

_EPS_KEYS = ("rms_norm_eps", "layer_norm_eps", "norm_epsilon", "layer_norm_epsilon", "norm_eps", "layernorm_epsilon")


@dataclass(frozen=True)
class RopeScaling:
    """`kind` is one of "none", "linear", "llama3", "yarn", "longrope".

    yarn (plan.rs:1433-1477 → config.rs:1558-1569): `extrapolation`, `attention`, `beta_fast`, `beta_slow`,
    `truncate` are the values the reference's engine reads, with its defaults; `attention` is the checkpoint's
    magnitude of cos and sin (`attention_factor`, or the quotient of the `mscale` pair), None for the built-in
    1 + 0.1 ln(factor).  longrope (plan.rs:1507-1548): per-lane divisors for
    contexts up to `original_max_position` (`short_factor`) and beyond (`long_factor`); `attention` multiplies
    cos and sin.  `dynamic` with an `alpha` only changes the base (plan.rs:1339-1343) and leaves kind "none".
    """

    kind: str = "none"
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position: int = 0
    extrapolation: float = 1.0
    attention: Optional[float] = None
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    truncate: bool = True
    short_factor: Tuple[float, ...] = ()
    long_factor: Tuple[float, ...] = ()


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    rope_dims: int
    rope_scaling: RopeScaling
    max_position: int
    tie_word_embeddings: bool
    # window[i] is the number of keys layer i sees (itself included), None for all keys
    layer_windows: Tuple[Optional[int], ...]
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    model_type: str = "llama"

    @staticmethod
    def from_json_file(path: str) -> "LlamaConfig":
        return LlamaConfig.from_dict(read_config_json(path))

    @staticmethod
    def from_dict(cfg: Dict[str, Any]) -> "LlamaConfig":
        if cfg.get("quantization_config") is not None:
            raise ConfigError("quantized checkpoints (quantization_config) are not supported")
        hidden = _uint(cfg, "hidden_size")
        if hidden is None:
            raise ConfigError("config.json requires valid hidden_size")
        heads = _uint(cfg, "num_attention_heads")
        if heads is None:
            raise ConfigError("config.json requires valid num_attention_heads")
        layers = _first(_uint(cfg, "num_hidden_layers"), _uint(cfg, "num_layers"))
        if layers is None:
            raise ConfigError("config.json requires valid num_hidden_layers")
        inter = _first(_uint(cfg, "intermediate_size"), _uint(cfg, "ffn_hidden_size"))
        if inter is None:
            raise ConfigError("config.json requires valid intermediate_size")
        kv_heads = _first(_uint(cfg, "num_key_value_heads"), heads)
        explicit_head_dim = _first(_uint(cfg, "head_dim"), _uint(cfg, "kv_channels"))
        if hidden == 0 or heads == 0 or layers == 0 or inter == 0 or kv_heads == 0:
            raise ConfigError("invalid or inconsistent model dimensions in config.json")
        if explicit_head_dim is None and hidden % heads != 0:
            raise ConfigError("invalid or inconsistent model dimensions in config.json")
        head_dim = explicit_head_dim if explicit_head_dim is not None else hidden // heads
        if head_dim == 0:
            raise ConfigError("invalid or inconsistent model dimensions in config.json")
        if heads % kv_heads != 0:
            raise ConfigError(f"head count {heads} is not a multiple of key/value head count {kv_heads}")
        vocab = _first(_uint(cfg, "vocab_size"), 32000)
        if vocab == 0:
            raise ConfigError("invalid or inconsistent model dimensions in config.json")
        max_position = _first(_uint(cfg, "max_position_embeddings"), _uint(cfg, "seq_length"), 40960)
        if max_position == 0:
            raise ConfigError("invalid or inconsistent model dimensions in config.json")

        activation = str(cfg.get("hidden_act", "silu")).lower()
        if activation not in ("silu", "swish"):
            raise ConfigError(f"unsupported activation {activation!r}; llama uses silu")

        eps = None
        for key in _EPS_KEYS:
            eps = _float(cfg, key)
            if eps is not None:
                break
        if eps is None:
            eps = 1e-6
        if not math.isfinite(eps) or eps <= 0.0:
            raise ConfigError("invalid rms_norm_eps")

        rope_raw, rope_kind, theta = _rope_params(cfg)
        if theta is None:
            theta = 10000.0
        if not math.isfinite(theta) or theta <= 0.0:
            raise ConfigError("invalid rope_theta")
        partial = _first(_float(rope_raw, "partial_rotary_factor"), _float(cfg, "partial_rotary_factor"))
        rope_dims = head_dim
        if partial is not None and abs(partial - 1.0) > 1e-9:
            rope_dims = int(round(head_dim * partial))
        if head_dim % 2 != 0 or rope_dims % 2 != 0 or rope_dims <= 0 or rope_dims > head_dim:
            raise ConfigError("the decoder requires even head and rotary dimensions")
        if rope_kind == "dynamic" and _float(rope_raw, "alpha") is not None:
            # plan.rs:1339-1343: the NTK-aware base; nothing else of the scaling is kept (:1376)
            theta = theta * _float(rope_raw, "alpha") ** (head_dim / (head_dim - 2.0))
            scaling = RopeScaling()
        else:
            scaling = _rope_scaling(rope_raw, rope_kind, cfg, rope_dims, max_position)

        windows = _layer_windows(cfg, layers)

        eos = cfg.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, list):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        bos = cfg.get("bos_token_id")
        return LlamaConfig(
            hidden_size=hidden,
            num_layers=layers,
            num_heads=heads,
            num_kv_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=inter,
            vocab_size=vocab,
            rms_norm_eps=float(eps),
            rope_theta=float(theta),
            rope_dims=rope_dims,
            rope_scaling=scaling,
            max_position=max_position,
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            layer_windows=windows,
            eos_token_ids=eos_ids,
            bos_token_id=int(bos) if isinstance(bos, int) else None,
        )

    def to_dict(self) -> Dict[str, Any]:
        """config.json content that `from_dict` reads back to an equal configuration."""
        out: Dict[str, Any] = {
            "model_type": "llama",
            "architectures": ["LlamaForCausalLM"],
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position,
            "hidden_act": "silu",
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.rope_dims != self.head_dim:
            out["partial_rotary_factor"] = self.rope_dims / self.head_dim
        s = self.rope_scaling
        if s.kind == "linear":
            out["rope_scaling"] = {"rope_type": "linear", "factor": s.factor}
        elif s.kind == "llama3":
            out["rope_scaling"] = {
                "rope_type": "llama3",
                "factor": s.factor,
                "low_freq_factor": s.low_freq_factor,
                "high_freq_factor": s.high_freq_factor,
                "original_max_position_embeddings": s.original_max_position,
            }
        elif s.kind == "yarn":
            out["rope_scaling"] = {
                "rope_type": "yarn",
                "factor": s.factor,
                "original_max_position_embeddings": s.original_max_position,
                "beta_fast": s.beta_fast,
                "beta_slow": s.beta_slow,
                "extrapolation_factor": s.extrapolation,
                "truncate": s.truncate,
            }
            if s.attention is not None:
                out["rope_scaling"]["attention_factor"] = s.attention
        elif s.kind == "longrope":
            out["rope_scaling"] = {
                "rope_type": "longrope",
                "short_factor": list(s.short_factor),
                "long_factor": list(s.long_factor),
                "original_max_position_embeddings": s.original_max_position,
                "attention_factor": s.attention,
            }
        windows = [w for w in self.layer_windows if w is not None]
        if windows:
            out["sliding_window"] = windows[0]
            out["layer_types"] = ["sliding_attention" if w is not None else "full_attention" for w in self.layer_windows]
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out


def _first(*values):
    for v in values:
        if v is not None:
            return v
    return None


def _uint(cfg: Any, key: str) -> Optional[int]:
    if not isinstance(cfg, dict):
        return None
    v = cfg.get(key)
    if isinstance(v, bool) or v is None:
        return None
    if isinstance(v, int) and v >= 0:
        return v
    if isinstance(v, float) and v >= 0 and v == int(v):
        return int(v)
    return None


def _float(cfg: Any, key: str) -> Optional[float]:
    if not isinstance(cfg, dict):
        return None
    v = cfg.get(key)
    if isinstance(v, bool) or v is None:
        return None
    if isinstance(v, (int, float)):
        return float(v)
    return None


def _rope_params(cfg: Dict[str, Any]) -> Tuple[Dict[str, Any], str, Optional[float]]:
    """The rotary parameter object, its kind and the base, from either `rope_parameters` (new
    form, possibly keyed by layer type) or `rope_scaling` (old form).  plan.rs:92-121."""
    raw: Any = None
    p = cfg.get("rope_parameters")
    if isinstance(p, dict):
        per_layer = p.get("full_attention")
        if isinstance(per_layer, dict):
            raw = per_layer
        elif "rope_type" in p or "rope_theta" in p:
            raw = p
        else:
            raw = next((v for v in p.values() if isinstance(v, dict)), None)
    if raw is None:
        s = cfg.get("rope_scaling")
        raw = s if isinstance(s, dict) else {}
    kind = raw.get("rope_type", raw.get("type", "default"))
    kind = str(kind).lower() if isinstance(kind, str) else "default"
    theta = _first(_float(raw, "rope_theta"), _float(cfg, "rope_theta"))
    return raw, kind, theta


def _rope_scaling(raw: Dict[str, Any], kind: str, cfg: Dict[str, Any], rope_dims: int, ctx: int) -> RopeScaling:
    if kind == "default":
        return RopeScaling()
    if kind == "linear":
        factor = _float(raw, "factor")
        if factor is None:
            raise ConfigError("linear rope_scaling requires factor")
        if not factor > 0.0:
            raise ConfigError("invalid rope_scaling factor")
        return RopeScaling(kind="linear", factor=factor)
    if kind == "llama3":
        factor = _float(raw, "factor")
        if factor is None:
            raise ConfigError("llama3 rope_scaling requires factor")
        original = _float(raw, "original_max_position_embeddings")
        if original is None:
            raise ConfigError("llama3 rope_scaling requires original_max_position_embeddings")
        low = _first(_float(raw, "low_freq_factor"), 1.0)
        high = _first(_float(raw, "high_freq_factor"), 4.0)
        if not factor > 0.0 or not original > 0.0 or low == high:
            raise ConfigError("invalid llama3 rope_scaling values")
        return RopeScaling(kind="llama3", factor=factor, low_freq_factor=low, high_freq_factor=high,
                           original_max_position=int(original))
    if kind == "yarn":
        # plan.rs:1433-1477 (config.json keys) and config.rs:1558-1569 (the engine's defaults)
        factor = _float(raw, "factor")
        if factor is None:
            raise ConfigError("yarn rope_scaling requires factor")
        original = _first(_uint(raw, "original_max_position_embeddings"), _uint(cfg, "original_max_position_embeddings"))
        if original is None:
            raise ConfigError("yarn rope_scaling requires original_max_position_embeddings")
        if not factor > 0.0 or original == 0:
            raise ConfigError("invalid yarn rope_scaling values")
        magnitude = lambda m: 0.1 * m * math.log(factor) + 1.0
        given = _float(raw, "attention_factor")
        if given is None:
            a, b = _float(raw, "mscale"), _float(raw, "mscale_all_dim")
            if a is not None and b is not None:
                given = magnitude(a) / magnitude(b)
        return RopeScaling(kind="yarn", factor=factor, original_max_position=original, attention=given,
                           beta_fast=_first(_float(raw, "beta_fast"), 32.0),
                           beta_slow=_first(_float(raw, "beta_slow"), 1.0),
                           extrapolation=_first(_float(raw, "extrapolation_factor"), 1.0),
                           truncate=raw.get("truncate") is not False)
    if kind in ("longrope", "su"):
        # plan.rs:1507-1548
        def factors(key: str) -> Tuple[float, ...]:
            v = raw.get(key)
            if not isinstance(v, list):
                raise ConfigError(f"longrope scaling requires {key}")
            return tuple(float(x) for x in v if isinstance(x, (int, float)) and not isinstance(x, bool))
        short, long = factors("short_factor"), factors("long_factor")
        lanes = rope_dims // 2
        if len(short) != lanes or len(long) != lanes:
            raise ConfigError(f"longrope factors must have {lanes} entries")
        original = _first(_uint(raw, "original_max_position_embeddings"), _uint(cfg, "original_max_position_embeddings"), ctx)
        if original == 0 or any(not f > 0.0 for f in short + long):
            raise ConfigError("invalid longrope scaling values")
        scale = ctx / original
        default = math.sqrt(1.0 + math.log(scale) / math.log(original)) if scale > 1.0 else 1.0
        return RopeScaling(kind="longrope", original_max_position=original,
                           attention=_first(_float(raw, "attention_factor"), default),
                           short_factor=short, long_factor=long)
    if kind in ("dynamic", "dynamic-ntk", "dynamic_ntk"):
        # the reference's planner passes the kind on (plan.rs:1379-1392) and its engine then refuses the model
        # with these words (rust/engine/src/config.rs:1570); only `dynamic` with an `alpha` runs (above)
        raise ConfigError('unsupported rope scaling type "dynamic"')
    raise ConfigError(f"unsupported rope_scaling type {kind!r}")


def _layer_windows(cfg: Dict[str, Any], layers: int) -> Tuple[Optional[int], ...]:
    """plan.rs:1239-1287: a positive `sliding_window` applies unless `use_sliding_window` is
    false; `layer_types` of the right length chooses the layers, otherwise every layer."""
    window = _uint(cfg, "sliding_window")
    if not window:
        return tuple([None] * layers)
    if cfg.get("use_sliding_window") is False:
        return tuple([None] * layers)
    types = cfg.get("layer_types")
    if isinstance(types, list) and len(types) == layers:
        return tuple(window if t == "sliding_attention" else None for t in types)
    return tuple([window] * layers)
