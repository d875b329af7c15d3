"""The step function: one batch of (request, its next tokens) in, logits at the wanted places out.

`ModelRunner` owns the model, the cache manager and the device pages.  `step` runs exactly the
tokens it is given, as one batch, against what earlier steps left in the cache: portions of
prompts beside single decoded tokens, cut anywhere.  Everything above (scheduler, generation,
trace replay) goes through it.  The reference's counterpart is `RustDecoder::forward`
(rust/engine/src/rust_decoder.rs:8378-8398; batch validation :8551-8578; how the runtime builds
a batch: rust/engine/src/runtime.rs:2380-2442).
"""
from __future__ import annotations

import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache import CacheManager, OutOfPages
from ..config.llama import read_config_json
from ..config.spec import ModelSpec
from ..parts.runtime import Runtime
from ..registry import model_spec_from_config
from ..weights.loader import check_tensors, load_checkpoint
from .context import StepContext
from .model import Model

_DTYPES = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
           "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}


def parse_dtype(name: Union[str, torch.dtype]) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.float32, torch.bfloat16):
            raise ValueError(f"dtype must be float32 or bfloat16, not {name}")
        return name
    try:
        return _DTYPES[name.lower()]
    except KeyError:
        raise ValueError(f"dtype must be float32 or bfloat16, not {name!r}") from None


class StepError(ValueError):
    """A batch the step function refuses before anything is launched."""


@dataclass
class StepEntry:
    """A request's next tokens.  `want`: indices into `tokens` whose logits are returned."""
    req_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()


class ModelRunner:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype="bfloat16", device="cuda:0",
                 page_size: int = 16, max_tokens: Optional[int] = None, num_pages: Optional[int] = None,
                 max_requests: int = 16, max_context: Optional[int] = None, memory_utilization: float = 0.90,
                 ops=None, typed_config=None):
        self.spec = spec
        self.config = typed_config
        self.device = torch.device(device)
        self.dtype = parse_dtype(dtype)
        if ops is None:
            from ..kernels import Ops
            ops = Ops()
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        self.page_size = page_size
        self.max_context = int(min(max_context or spec.max_position, spec.max_position))
        self.rt = Runtime(self.device, self.dtype, ops, self.max_context)
        check_tensors(spec, {n: tuple(t.shape) for n, t in tensors.items()})
        self.model = Model(spec, tensors, self.rt)
        self.vocab_size = spec.vocab_size
        num_groups = len(self.model.group_keys)
        if num_pages is None and max_tokens is not None:
            num_pages = -(-int(max_tokens) // page_size)
        if num_pages is None:
            num_pages = self._pages_that_fit(memory_utilization, max_requests)
        if num_pages <= 0:
            raise ValueError("the cache needs at least one page")
        self.num_pages = int(num_pages)
        self.max_requests = max_requests
        self.cache: CacheManager = self.model.allocate_caches(page_size, [self.num_pages] * num_groups, max_requests)
        self.steps = 0
        self.rows_total = 0

    # ---- construction ---------------------------------------------------------------------
    @staticmethod
    def from_folder(model_dir: str, **kwargs) -> "ModelRunner":
        """The model class is chosen by config.json; weights are bound by tensor name."""
        config = read_config_json(model_dir)
        typed, spec = model_spec_from_config(config)
        tensors = load_checkpoint(model_dir, spec)
        return ModelRunner(spec, tensors, typed_config=typed, **kwargs)

    def _pages_that_fit(self, utilization: float, max_requests: int) -> int:
        """Pages for what is left of the card after the weights, capped at what `max_requests`
        requests of full context can use."""
        per_page = max(1, self.model.cache_bytes_per_page(self.page_size))
        cap = max_requests * (-(-self.max_context // self.page_size))
        if self.device.type != "cuda":
            return cap
        free, total = torch.cuda.mem_get_info(self.device)
        budget = int(free - (1.0 - utilization) * total) - (2 << 30)   # room for activations and logits
        return max(1, min(cap, budget // per_page))

    # ---- requests -------------------------------------------------------------------------
    def add_request(self, req_id) -> int:
        return self.cache.add_request(req_id)

    def free_request(self, req_id) -> None:
        self.cache.free_request(req_id)

    def length(self, req_id) -> int:
        return self.cache.length(req_id)

    # ---- the step -------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        if len(entries) > self.max_requests:
            raise StepError(f"{len(entries)} entries in one step, the engine holds at most {self.max_requests} requests")
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise StepError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.req_id!r} brings no tokens")
            for t in e.tokens:
                if not 0 <= int(t) < self.vocab_size:
                    raise StepError(f"token id {t} of request {e.req_id!r} is outside [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.req_id!r} wants logits at {w}, it brings {n} tokens")
            start = self.cache.length(e.req_id) if self.cache.has_request(e.req_id) else 0
            if start + n > self.max_context:
                raise StepError(f"request {e.req_id!r} would hold {start + n} tokens, the context is {self.max_context}")

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Runs the entries as one batch and returns float32 logits [wanted, vocab] on the device,
        in the order of the entries and of each entry's `want`.  Unknown requests are added.
        Raises `OutOfPages` (nothing changed) when the pages do not suffice."""
        self._validate(entries)
        added = []
        try:
            for e in entries:
                if not self.cache.has_request(e.req_id):
                    self.cache.add_request(e.req_id)
                    added.append(e.req_id)
            # preflight over the whole batch, then reserve: a failure leaves no request changed
            need = [0] * len(self.cache.groups)
            for e in entries:
                total = self.cache.length(e.req_id) + len(e.tokens)
                for g, m in enumerate(self.cache.pages_missing(e.req_id, total)):
                    need[g] += m
            for g, n in enumerate(need):
                if n > self.cache.free_pages(g):
                    raise OutOfPages(f"the step needs {n} pages of cache group {g}, {self.cache.free_pages(g)} are free")
            for e in entries:
                self.cache.reserve(e.req_id, self.cache.length(e.req_id) + len(e.tokens))
        except Exception:
            for r in added:
                self.cache.free_request(r)
            raise
        ctx = self._build_context(entries)
        logits = self.model.forward(ctx)
        for e in entries:
            self.cache.commit(e.req_id, len(e.tokens))
        self.steps += 1
        self.rows_total += ctx.num_rows
        return logits

    def _build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        ids: List[int] = []
        row_pos: List[int] = []
        row_seg: List[int] = []
        slots: List[int] = []
        logit_rows: List[int] = []
        seg_rows, seg_start = [], []
        max_context = 0
        for s, e in enumerate(entries):
            start = self.cache.length(e.req_id)
            n = len(e.tokens)
            base = len(ids)
            ids.extend(int(t) for t in e.tokens)
            row_pos.extend(range(start, start + n))
            row_seg.extend([s] * n)
            slots.append(self.cache.slot(e.req_id))
            logit_rows.extend(base + int(w) for w in e.want)
            seg_rows.append(n)
            seg_start.append(start)
            max_context = max(max_context, start + n)
        S = len(entries)
        widths = []
        flat_tables: List[int] = []
        for g in range(len(self.cache.groups)):
            width = max(1, max(len(self.cache.table(e.req_id, g)) for e in entries))
            widths.append(width)
            for e in entries:
                t = self.cache.table(e.req_id, g)
                flat_tables.extend(t)
                flat_tables.extend([-1] * (width - len(t)))
        cu_rows = [0]
        for n in seg_rows:
            cu_rows.append(cu_rows[-1] + n)
        packed = torch.tensor(ids + row_pos + row_seg + cu_rows + slots + logit_rows + flat_tables, dtype=torch.int32)
        packed = packed.to(self.device, non_blocking=False)
        R, L = len(ids), len(logit_rows)
        o = 0

        def take(count):
            nonlocal o
            out = packed[o:o + count]
            o += count
            return out

        t_ids, t_pos, t_seg, t_cu, t_slots, t_rows = take(R), take(R), take(R), take(S + 1), take(S), take(L)
        tables = [take(S * w).view(S, w) for w in widths]
        return StepContext(num_rows=R, num_segments=S, ids=t_ids, row_pos=t_pos, row_seg=t_seg, seg_start=t_cu,
                           slots=t_slots,
                           logit_rows=t_rows, tables=tables, seg_rows=seg_rows, seg_pos_start=seg_start,
                           seg_slots=slots, max_context=max_context, uniform_rows=all(n == 1 for n in seg_rows))
