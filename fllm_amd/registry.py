"""Registries: architecture name -> model description, and part kind -> part class.

Adding an architecture or a part never edits this file: the new module calls `register_*` when it
is imported (tests register toy parts the same way).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Sequence

from .config.spec import ConfigError, ModelSpec


@dataclass(frozen=True)
class Architecture:
    model_type: str
    hf_architectures: Sequence[str]
    parse_config: Callable[[Dict[str, Any]], Any]      # config.json dict -> typed config
    build_spec: Callable[[Any], ModelSpec]              # typed config -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}
_PARTS: Dict[str, Dict[str, type]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {},
                                      "embedding": {}, "head": {}}


def register_architecture(arch: Architecture) -> None:
    _ARCHITECTURES[arch.model_type.lower()] = arch


def supported_model_types() -> List[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(config: Dict[str, Any]) -> Architecture:
    """Dispatch on `model_type` (lower-cased), as the reference's decoders do
    (rust/checkpoint/src/plan.rs:880-884, :972-974); `architectures`, when present, must agree."""
    raw = config.get("model_type")
    if not isinstance(raw, str) or not raw:
        raise ConfigError("config.json requires model_type")
    arch = _ARCHITECTURES.get(raw.lower())
    if arch is None:
        raise ConfigError(f"unsupported model_type {raw!r}; refusing fallback architecture mapping "
                          f"(supported: {', '.join(supported_model_types())})")
    named = config.get("architectures")
    if isinstance(named, list) and named and arch.hf_architectures:
        if not any(n in arch.hf_architectures for n in named):
            raise ConfigError(f"model_type {raw!r} does not match architectures {named!r} "
                              f"(expected one of {list(arch.hf_architectures)!r})")
    return arch


def model_spec_from_config(config: Dict[str, Any]):
    """(typed config, ModelSpec) of a config.json dict."""
    arch = resolve_architecture(config)
    typed = arch.parse_config(config)
    spec = arch.build_spec(typed)
    spec.validate()
    return typed, spec


def register_part(role: str, kind: str, cls: type) -> None:
    if role not in _PARTS:
        raise KeyError(f"unknown part role {role!r}; roles: {sorted(_PARTS)}")
    _PARTS[role][kind] = cls


def part_class(role: str, kind: str) -> type:
    try:
        return _PARTS[role][kind]
    except KeyError:
        raise ConfigError(f"no {role} part of kind {kind!r} is registered "
                          f"(registered: {sorted(_PARTS.get(role, {}))})") from None
