"""A model put together from parts as its `ModelSpec` says, and the plan of its caches."""
from __future__ import annotations

import math
from typing import Dict, List, NamedTuple, Optional, Sequence, Tuple

import torch

from ..cache import CacheManager, GroupSpec
from ..config.spec import ModelSpec
from ..parts.base import KVNeed, StateNeed
from ..parts.runtime import Runtime
from ..registry import part_class
from ..weights.loader import part_weights
from .context import CacheBinding, StepContext


class GroupKey(NamedTuple):
    """What run entries must have in common to share the pages of one cache group."""
    kv_heads: int
    k_dim: int
    v_dim: int
    window: Optional[int]
    key_chunk: int


class Model:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], rt: Runtime, consume_tensors: bool = False):
        spec.validate()
        self.spec = spec
        self.rt = rt

        def make(role, part, **extra):
            return part_class(role, part.kind)(part, part_weights(part, tensors), rt, **extra)

        rt.collect_tile_requests()       # copies of matrices for decode steps are made when all weights are placed
        self.embedding = make("embedding", spec.embedding)
        self.blocks = []
        for layer in spec.layers:
            norms = {name: make("norm", n) for name, n in layer.norms.items()}
            mixer = make("mixer", layer.mixer)
            ffn = make("feed_forward", layer.feed_forward) if layer.feed_forward is not None else None
            placed = dict(mixer=mixer, feed_forward=ffn, norms=norms)
            if layer.extras:            # only an arrangement that names further parts is handed them
                placed["extras"] = {name: make(role, part) for name, (role, part) in layer.extras.items()}
            self.blocks.append(make("block", layer.block, **placed))
        self.final_norm = make("norm", spec.final_norm)
        self.head = make("head", spec.head)
        if consume_tensors:
            tensors.clear()              # the parts hold what they use; what they joined into one matrix is given back
        self.decode_tile_bytes = rt.tiles_for_model()
        self.bindings: List[CacheBinding] = []
        self.layer_check = None          # a diagnostics.LayerCheck while layers are being checked
        self._plan_caches()

    # ---- caches ---------------------------------------------------------------------------
    def _plan_caches(self) -> None:
        """Groups cache-owning run entries by what they need; entries that read another entry's
        cache join that entry's group."""
        self.kv_needs: List[Optional[KVNeed]] = []
        self.state_needs: List[object] = []          # per run entry None, a StateNeed, or a dict of named ones
        self.portion_multiple = 1                    # a prompt is cut on multiples of every mixer's own multiple
        for entry in self.spec.run_order:
            mixer = self.blocks[entry.layer].mixer
            self.kv_needs.append(mixer.cache_need())
            self.state_needs.append(mixer.state_need())
            multiple = int(getattr(mixer, "portion_multiple", lambda: 1)())
            if multiple <= 0:
                raise ValueError(f"run entry of layer {entry.layer}: portion_multiple() must be positive, is {multiple}")
            self.portion_multiple = self.portion_multiple * multiple // math.gcd(self.portion_multiple, multiple)
        keys: List[GroupKey] = []
        self.entry_group: List[Optional[int]] = [None] * len(self.spec.run_order)
        self.entry_index: List[Optional[int]] = [None] * len(self.spec.run_order)   # index inside the group's tensors
        members: List[List[int]] = []
        for i, entry in enumerate(self.spec.run_order):
            need = self.kv_needs[i]
            if need is None:
                continue
            if entry.reads_cache_of is not None:
                src = entry.reads_cache_of
                src_need = self.kv_needs[src]
                if src_need is None or ((src_need.kv_heads, src_need.k_dim, src_need.v_dim, src_need.key_chunk)
                                        != (need.kv_heads, need.k_dim, need.v_dim, need.key_chunk)):
                    raise ValueError(f"run entry {i} cannot read the cache of entry {src}: different geometry")
                if src_need.window is not None and (need.window is None or need.window > src_need.window):
                    raise ValueError(f"run entry {i} needs more keys than entry {src} keeps")
                self.entry_group[i] = self.entry_group[src]
                self.entry_index[i] = self.entry_index[src]
                continue
            key = GroupKey(need.kv_heads, need.k_dim, need.v_dim, need.window, need.key_chunk)
            if key not in keys:
                keys.append(key)
                members.append([])
            g = keys.index(key)
            self.entry_group[i] = g
            self.entry_index[i] = len(members[g])
            members[g].append(i)
        self.group_keys = keys
        self.group_members = members

    def group_specs(self, page_size: int) -> List[GroupSpec]:
        return [GroupSpec(entries=tuple(m), kv_heads=k.kv_heads, k_dim=k.k_dim, v_dim=k.v_dim, window=k.window, page_size=page_size)
                for k, m in zip(self.group_keys, self.group_members)]

    def cache_bytes_per_page(self, page_size: int) -> List[int]:
        """Bytes a page of each group costs (keys and values of all the group's run entries)."""
        elem = torch.empty((), dtype=self.rt.dtype).element_size()
        return [len(m) * k.kv_heads * (k.k_dim + k.v_dim) * page_size * elem for k, m in zip(self.group_keys, self.group_members)]

    def allocate_caches(self, page_size: int, pages_per_group: Sequence[int], max_requests: int,
                        max_step_tokens: Optional[int] = None) -> CacheManager:
        """Device pages for every group (one page more than the manager hands out: the null page
        that padding rows of a captured step write to) and the state arenas."""
        rt = self.rt
        groups = self.group_specs(page_size)
        if len(pages_per_group) != len(groups):
            raise ValueError(f"{len(groups)} cache groups need {len(groups)} page counts")
        self.page_size = page_size
        self.null_pages = [int(n) for n in pages_per_group]
        self.k_store, self.v_store = [], []
        for g, n in zip(groups, pages_per_group):
            need = self.kv_needs[g.entries[0]]            # the group's entries agree on what they need
            self.k_store.append(torch.zeros((len(g.entries), n + 1, g.kv_heads, *need.key_page_shape(page_size)),
                                            dtype=rt.dtype, device=rt.device))
            self.v_store.append(torch.zeros((len(g.entries), n + 1, g.kv_heads, g.v_dim, page_size),
                                            dtype=rt.dtype, device=rt.device))
        self.bindings = []
        for i, entry in enumerate(self.spec.run_order):
            g = self.entry_group[i]
            arena = lambda need: torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=rt.device)
            need = self.state_needs[i]
            state = None if need is None else ({name: arena(n) for name, n in need.items()} if isinstance(need, dict)
                                               else arena(need))
            if g is None:
                self.bindings.append(CacheBinding(group=-1, k_pages=None, v_pages=None, page_size=page_size,
                                                  writes=False, state=state))
                continue
            idx = self.entry_index[i]
            self.bindings.append(CacheBinding(group=g, k_pages=self.k_store[g][idx], v_pages=self.v_store[g][idx],
                                              page_size=page_size, writes=entry.reads_cache_of is None, state=state))
        return CacheManager(groups, list(pages_per_group), max_requests, max_step_tokens=max_step_tokens)

    def state_arenas(self):
        """(run entry, name or None, arena [max_requests, *shape]) of every state tensor the model keeps."""
        for index, binding in enumerate(self.bindings):
            if isinstance(binding.state, dict):
                for name, arena in binding.state.items():
                    yield index, name, arena
            elif binding.state is not None:
                yield index, None, binding.state

    def clear_state(self, slot: int) -> None:
        """Zeros the fixed-size state of every run entry in one request slot (a request's first step)."""
        for _, _, arena in self.state_arenas():
            arena[slot].zero_()

    def snapshot_state(self, slot: int):
        """A copy of everything the model keeps in one request slot, for `restore_state`
        (the reference's sequence state snapshots, rust/engine/src/rust_decoder/state_api.rs:14-80)."""
        return [(index, name, arena[slot].clone()) for index, name, arena in self.state_arenas()]

    def restore_state(self, slot: int, snapshot) -> None:
        """Puts a snapshot (of this model, of any slot) into `slot`."""
        arenas = {(index, name): arena for index, name, arena in self.state_arenas()}
        if sorted(arenas, key=str) != sorted(((i, n) for i, n, _ in snapshot), key=str):
            raise ValueError("the snapshot is not one of this model's state")
        for index, name, saved in snapshot:
            arenas[(index, name)][slot].copy_(saved)

    @property
    def has_state(self) -> bool:
        return any(b.state is not None for b in self.bindings)

    # ---- forward --------------------------------------------------------------------------
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """Logits (float32 [len(logit_rows), vocab]) of the step's wanted rows."""
        x = self.embedding.forward(ctx, ctx.ids)
        pending = None      # a block's output that the next block adds together with its first norm
        check = self.layer_check if self.layer_check is not None and self.layer_check.active else None
        order = self.spec.run_order
        for index, (entry, binding) in enumerate(zip(order, self.bindings)):
            block = self.blocks[entry.layer]
            if check is not None:
                check.run_block(self, block, ctx, x, binding, index, entry.layer)
                continue
            # the norm that reads the residual stream after this block: the first one of the block that runs next,
            # where that block says which it is (a block may let its last sum prepare it)
            ctx.next_norm = self.blocks[order[index + 1].layer].first_norm() if index + 1 < len(order) else None
            if getattr(block, "takes_pending", False):
                pending = block.forward(ctx, x, binding, pending)
            else:
                if pending is not None:
                    self.rt.ops.add_residual(x, pending)
                pending = None
                block.forward(ctx, x, binding)
        ctx.next_norm = ctx.prepared = None
        if pending is not None:
            self.rt.ops.add_residual(x, pending)
        if check is not None:
            check.end_step()
        if ctx.logit_rows.numel() == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=self.rt.device)
        h = self.final_norm.forward(ctx, x, rows=ctx.logit_rows)
        return self.head.forward(ctx, h)
