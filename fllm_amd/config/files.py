"""Reading a checkpoint's config.json, whatever architecture it describes."""
from __future__ import annotations

import json
import os
from typing import Any, Dict

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
