"""Reading a checkpoint's config.json, whatever architecture it describes."""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Optional, Tuple

from .spec import ConfigError


def read_config_json(path: str) -> Dict[str, Any]:
    """`path` is a model folder or a config.json file."""
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            cfg = json.load(fh)
    except FileNotFoundError:
        raise ConfigError(f"{path} not found") from None
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path} is not valid JSON: {exc}") from None
    if not isinstance(cfg, dict):
        raise ConfigError(f"{path} must hold a JSON object")
    return cfg


_GENERATION_RANGES = {"temperature": (0.0, 100.0), "top_p": (0.0, 1.0), "min_p": (0.0, 1.0), "repetition_penalty": (0.0001, 100.0)}


def generation_defaults(source: str, model_dir: Optional[str]) -> Tuple[Dict[str, Any], str]:
    """Sampling defaults that ship with a model (rust/engine/src/server/gencfg.rs:93-135): `source` is `auto` (the
    generation_config.json in the model folder, if there is one), `vllm` (none) or a path to such a file or to a
    folder that holds one.  Of the file's keys temperature, top_p, top_k, min_p and repetition_penalty are taken,
    whether or not `do_sample` is set; values a sampler cannot use are dropped rather than refused (:68-79), numbers
    are rounded to six digits, a `top_k` of 0 or below means off.  A file named outright must be readable; with
    `auto` a missing or broken one means no defaults.  Returns (defaults, where they came from)."""
    source = source.strip()
    if source == "vllm":
        return {}, "none (--generation-config vllm)"
    explicit = source != "auto"
    path = source if explicit else model_dir
    if path is None:
        return {}, "none in the model"
    if os.path.isdir(path):
        path = os.path.join(path, "generation_config.json")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            value = json.load(fh)
        if not isinstance(value, dict):
            raise ValueError("not a JSON object")
    except (OSError, ValueError) as exc:
        if explicit:
            raise ConfigError(f"cannot read generation defaults from {path}: {exc}") from None
        return {}, "none in the model"
    out: Dict[str, Any] = {}
    for key, (low, high) in _GENERATION_RANGES.items():
        v = value.get(key)
        if isinstance(v, (int, float)) and not isinstance(v, bool) and v == v and low <= v <= high:
            out[key] = round(float(v) * 1e6) / 1e6
    k = value.get("top_k")
    if isinstance(k, int) and not isinstance(k, bool) and k >= 0:
        out["top_k"] = k
    return out, (path if out or explicit else "none in the model")


def generation_eos_ids(model_dir: str) -> Tuple[int, ...]:
    """The end-of-sequence ids of a model folder's generation_config.json (one id or a list), for models whose
    config.json names none."""
    try:
        with open(os.path.join(model_dir, "generation_config.json"), "r", encoding="utf-8") as fh:
            eos = json.load(fh).get("eos_token_id")
    except (OSError, ValueError, AttributeError):
        return ()
    if isinstance(eos, int) and not isinstance(eos, bool):
        return (eos,)
    if isinstance(eos, list) and all(isinstance(e, int) and not isinstance(e, bool) for e in eos):
        return tuple(eos)
    return ()
