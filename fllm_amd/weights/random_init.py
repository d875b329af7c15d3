"""Random-weights mode: a model folder (config.json, model.safetensors) from a configuration and
a seed.

Distributions: matrices, embedding and biases N(0, 0.02); norm weights 1 + U(-0.1, 0.1).  (The
reference's own generator, rust/engine/src/tiny_model.rs:44-60 and :118-140, draws uniform
weights from one xorshift stream; here every tensor has a stream of its own, keyed by seed and
tensor name, so the values do not depend on the order in which tensors are made.)
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Dict

import torch

from ..config.spec import ModelSpec
from ..parts.base import INIT_BIAS, INIT_MATRIX, INIT_NORM
from ..registry import model_spec_from_config
from .loader import expected_tensors
from .safetensors_io import write_safetensors


def _generator(seed: int, name: str, device="cpu") -> torch.Generator:
    digest = hashlib.sha256(f"{seed}:{name}".encode("utf-8")).digest()
    g = torch.Generator(device=device)
    g.manual_seed(int.from_bytes(digest[:8], "little") & ((1 << 63) - 1))
    return g


def random_tensor(name: str, shape, kind: str, seed: int, dtype: torch.dtype, device="cpu") -> torch.Tensor:
    g = _generator(seed, name, device)
    if kind == INIT_NORM:
        t = 1.0 + (torch.rand(shape, generator=g, dtype=torch.float32, device=device) * 0.2 - 0.1)
    elif kind in (INIT_MATRIX, INIT_BIAS):
        t = torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, 0.02, generator=g)
    else:
        raise ValueError(f"unknown init kind {kind!r}")
    return t.to(dtype)


def random_tensors(spec: ModelSpec, seed: int, dtype: torch.dtype, device="cpu",
                   with_optional: bool = False) -> Dict[str, torch.Tensor]:
    """Every required tensor of the model (and the optional ones on request) by checkpoint name."""
    required, optional, init = expected_tensors(spec)
    names = dict(required)
    if with_optional:
        names.update(optional)
    return {n: random_tensor(n, shape, init[n], seed, dtype, device) for n, shape in names.items()}


def write_random_model(model_dir: str, config: Dict[str, Any], seed: int, dtype: str = "float32",
                       with_optional: bool = False) -> ModelSpec:
    """Writes `config` as config.json and seeded random tensors as model.safetensors."""
    torch_dtype = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}[dtype]
    _, spec = model_spec_from_config(config)
    os.makedirs(model_dir, exist_ok=True)
    cfg = dict(config)
    cfg.setdefault("torch_dtype", dtype)
    with open(os.path.join(model_dir, "config.json"), "w", encoding="utf-8") as fh:
        json.dump(cfg, fh, indent=1)
    write_safetensors(os.path.join(model_dir, "model.safetensors"),
                      random_tensors(spec, seed, torch_dtype, with_optional=with_optional))
    return spec
