"""Binding checkpoint tensors to the parts of a model by tensor name.

The parts say which tensors they take and with which shapes; the loader compares that with what
the checkpoint holds and reports everything that is wrong in ONE error: missing tensors,
unexpected tensors and wrong shapes (the reference reports these one at a time:
rust/checkpoint/src/convert.rs:560-572 shapes, :963-969 and :1280-1284 required tensors,
rust/checkpoint/src/plan.rs:3068-3093 unrecognised tensors).
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from ..config.spec import ModelSpec, PartSpec
from ..registry import part_class
from .safetensors_io import open_checkpoint


class WeightsError(ValueError):
    def __init__(self, missing: List[str], unexpected: List[str], wrong_shape: List[Tuple[str, tuple, tuple]]):
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        lines = ["checkpoint does not match the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(
                f"{n} has shape {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape))
        super().__init__("\n".join(lines))


def iter_parts(spec: ModelSpec):
    """(role, PartSpec) of every part of the model, each weight-holding part once."""
    yield "embedding", spec.embedding
    for layer in spec.layers:
        yield "block", layer.block
        for _, role, part in layer.parts():
            yield role, part
    yield "norm", spec.final_norm
    yield "head", spec.head


def expected_tensors(spec: ModelSpec):
    """(required, optional, init): checkpoint tensor name -> shape / init kind."""
    required: Dict[str, tuple] = {}
    optional: Dict[str, tuple] = {}
    init: Dict[str, str] = {}
    for role, part in iter_parts(spec):
        shapes = part_class(role, part.kind).tensor_shapes(part)
        for key, name in part.tensors.items():
            is_optional = key.startswith("?")
            param = key[1:] if is_optional else key
            if param not in shapes:
                raise KeyError(f"{role} part {part.kind!r} names tensor {param!r} but declares no shape for it")
            shape, kind = shapes[param]
            target = optional if is_optional else required
            if name in target and tuple(target[name]) != tuple(shape):
                raise ValueError(f"tensor {name} is bound twice with different shapes")
            target[name] = tuple(shape)
            init[name] = kind
    return required, optional, init


def canonical_names(spec: ModelSpec, names) -> Dict[str, str]:
    """Checkpoint tensor name -> the name the model knows it by, after the architecture's renaming rules
    (`ModelSpec.tensor_renames`); tensors under a skipped prefix are left out.  Two tensors that come to the same
    name are an error (the reference refuses duplicate targets, rust/checkpoint/src/plan.rs:3068-3093)."""
    out: Dict[str, str] = {}
    taken: Dict[str, str] = {}
    for name in names:
        canonical = name
        for prefix, replacement in spec.tensor_renames:
            if name.startswith(prefix):
                canonical = replacement + name[len(prefix):]
                break
        if any(canonical.startswith(p) for p in spec.skipped_tensor_prefixes):
            continue
        if canonical in taken:
            raise ValueError(f"checkpoint tensors {taken[canonical]!r} and {name!r} both stand for {canonical!r}")
        taken[canonical] = name
        out[name] = canonical
    return out


def check_tensors(spec: ModelSpec, shapes: Dict[str, tuple]) -> None:
    """Raises `WeightsError` unless `shapes` (name -> shape of what a checkpoint holds) fits."""
    required, optional, _ = expected_tensors(spec)
    ignorable = set(spec.ignorable_tensors)
    missing = [n for n in required if n not in shapes]
    unexpected = [n for n in shapes if n not in required and n not in optional and n not in ignorable]
    wrong = []
    for n, got in shapes.items():
        want = required.get(n, optional.get(n))
        if want is not None and tuple(got) != tuple(want):
            wrong.append((n, tuple(got), tuple(want)))
    if missing or unexpected or wrong:
        raise WeightsError(sorted(missing), sorted(unexpected), sorted(wrong))


def load_checkpoint(model_dir: str, spec: ModelSpec) -> Dict[str, torch.Tensor]:
    """Name -> CPU tensor in the stored dtype (views of the mapped files; integer tensors as
    int32) for every tensor the model takes."""
    stored = open_checkpoint(model_dir)
    found = {canonical: stored[name] for name, canonical in canonical_names(spec, stored).items()}
    check_tensors(spec, {n: f.entries[stored_name].shape for n, (f, stored_name) in found.items()})
    required, optional, _ = expected_tensors(spec)
    out: Dict[str, torch.Tensor] = {}
    for n in list(required) + [o for o in optional if o in found]:
        t = found[n][0].tensor(found[n][1])
        if not t.dtype.is_floating_point:
            t = t.to(torch.int32)
        out[n] = t
    return out


def part_weights(part: PartSpec, tensors: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The tensors of one part under the part's own parameter names (optional ones only if held)."""
    out = {}
    for key, name in part.tensors.items():
        if key.startswith("?"):
            if name in tensors:
                out[key[1:]] = tensors[name]
        else:
            out[key] = tensors[name]
    return out
