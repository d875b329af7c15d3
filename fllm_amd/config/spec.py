"""Architecture-neutral description of a model: what every layer is made of and in which
order layers run.

An architecture module turns its typed configuration into a `ModelSpec`.  Everything below the
architecture module (parts, cache manager, step function, loader) reads only the spec, so no part
knows which model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be loaded; raised before any weight is read."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: `kind` selects the class in the part registry, `params` are its sizes
    and constants, `tensors` maps the part's own parameter names to checkpoint tensor names."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    tensors: Dict[str, str] = field(default_factory=dict)

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]


@dataclass(frozen=True)
class LayerSpec:
    """A block: its arrangement (`block.kind`) and the parts the arrangement places.  `mixer` is the part that may own
    a cache or per-request state; `feed_forward` may be absent; `norms` are named by the arrangement; `extras` are
    further weight-holding parts of any role that the arrangement knows by name (name -> (role, PartSpec))."""

    block: PartSpec
    mixer: PartSpec
    feed_forward: Optional[PartSpec] = None
    norms: Dict[str, PartSpec] = field(default_factory=dict)
    extras: Dict[str, Tuple[str, PartSpec]] = field(default_factory=dict)

    def parts(self):
        """(name, role, PartSpec) of every part the layer places, the block's own spec aside."""
        for name, norm in self.norms.items():
            yield f"norm:{name}", "norm", norm
        yield "mixer", "mixer", self.mixer
        if self.feed_forward is not None:
            yield "feed_forward", "feed_forward", self.feed_forward
        for name, (role, part) in self.extras.items():
            yield f"extra:{name}", role, part


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  `layer` indexes `ModelSpec.layers` (a layer may be named by
    several entries: its weights run twice, each run with a cache of its own).  `reads_cache_of`
    names an earlier entry whose cache this entry reads instead of writing one."""

    layer: int
    reads_cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    run_order: Tuple[RunEntry, ...]
    final_norm: PartSpec
    head: PartSpec
    # tensor names a checkpoint may hold that do not affect the forward pass
    ignorable_tensors: Tuple[str, ...] = ()
    # checkpoints that nest the model under other names: (prefix, replacement) rules, the first that fits a tensor's
    # name applies; then tensors whose name begins with one of `skipped_tensor_prefixes` are left aside (towers of
    # other modalities beside the language model)
    tensor_renames: Tuple[Tuple[str, str], ...] = ()
    skipped_tensor_prefixes: Tuple[str, ...] = ()

    def validate(self) -> None:
        for i, entry in enumerate(self.run_order):
            if not 0 <= entry.layer < len(self.layers):
                raise ConfigError(f"run order entry {i} names layer {entry.layer}, model has {len(self.layers)}")
            src = entry.reads_cache_of
            if src is not None and not 0 <= src < i:
                raise ConfigError(f"run order entry {i} reads the cache of entry {src}, which does not run before it")
            if src is not None and self.run_order[src].reads_cache_of is not None:
                raise ConfigError(f"run order entry {i} reads the cache of entry {src}, which owns none")


def default_run_order(num_layers: int) -> Tuple[RunEntry, ...]:
    return tuple(RunEntry(layer=i) for i in range(num_layers))
