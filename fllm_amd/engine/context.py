"""What one step looks like to the parts: the rows of the batch and where their requests' caches are.

A batch is a list of segments (one per request in the step); segment s contributes
`seg_rows[s]` consecutive rows at positions seg_pos_start[s], seg_pos_start[s] + 1, ...
Row-level arrays say for each row its token, its position and its segment; segment-level
arrays give the block table per cache group and the state slot.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class CacheBinding:
    """Where one run entry keeps its keys and values (and state)."""
    group: int                              # index into StepContext.tables
    k_pages: Optional[torch.Tensor]         # [pages, kv_heads, *KVNeed.key_page_shape]: [page_size, k_dim], or chunked [k_dim / n, page_size, n]
    v_pages: Optional[torch.Tensor]         # [pages, kv_heads, v_dim, page_size]
    page_size: int
    writes: bool                            # False: the entry reads another entry's cache
    state: object = None                    # [max_requests, *shape], or name -> such a tensor: mixers with fixed-size state


@dataclass
class StepContext:
    num_rows: int
    num_segments: int
    ids: torch.Tensor                       # int32 [R]
    row_pos: torch.Tensor                   # int32 [R]
    row_seg: torch.Tensor                   # int32 [R]
    seg_start: torch.Tensor                 # int32 [S + 1]: first row of each segment, then R
    slots: torch.Tensor                     # int32 [S]
    logit_rows: torch.Tensor                # int32 [L]
    tables: List[torch.Tensor]              # per cache group: int32 [S, max_pages]
    # host copies, for parts that decide on the host
    seg_rows: List[int] = field(default_factory=list)
    seg_pos_start: List[int] = field(default_factory=list)
    seg_slots: List[int] = field(default_factory=list)
    max_context: int = 0                    # largest position + 1 in the step
    uniform_rows: bool = False              # every segment has exactly one row
    single_from: Optional[int] = None       # the segments from this one on have one row each (None: unknown)
    single_max_context: int = 0             # largest position + 1 among those single rows
    # A sum into the residual stream may prepare the norm that reads the stream next (`parts/base.py`, "a norm
    # prepared ahead"): whoever arranges the parts names that norm in `then_norm` before a part runs and in
    # `next_norm` for the part that ends a block; `prepared` is what the part left: (norm, residual stream, payload).
    then_norm: object = None
    next_norm: object = None
    prepared: object = None
    _scratch: Dict = field(default_factory=dict)

    def no_rotation(self, rt):
        """Rotary arguments of a mixer without position encoding: zero rotated lanes."""
        key = ("no_rotation", rt.device)
        if key not in rt.shared:
            empty = torch.zeros((1, 0), dtype=torch.float32, device=rt.device)
            rt.shared[key] = (empty, empty)
        cos, sin = rt.shared[key]
        return cos, sin, 0, 0

    def single_rows_from(self) -> int:
        """Index of the first segment from which every segment has one row."""
        if self.uniform_rows:
            return 0
        return self.num_segments if self.single_from is None else self.single_from

    def attention_workspace(self, rt, rows: int, heads: int, kv_heads: int, head_dim: int) -> Optional[torch.Tensor]:
        """Scratch for partial results of split contexts, one buffer per step shape: sized for the single rows of the
        step, which are the ones whose contexts are split."""
        singles = self.num_segments - self.single_rows_from()
        need = max(rt.ops.attention_workspace_bytes(n, heads, kv_heads, head_dim, self.max_context) for n in {rows, singles} if n > 0)
        if need == 0:
            return None
        buf = self._scratch.get("attention")
        if buf is None or buf.numel() < need:
            buf = torch.empty(need, dtype=torch.uint8, device=rt.device)
            self._scratch["attention"] = buf
        return buf
