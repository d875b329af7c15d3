"""The step function: one batch of (request, its next tokens) in, logits at the wanted places out.

`ModelRunner` owns the model, the cache manager and the device pages.  `step` runs exactly the
tokens it is given, as one batch, against what earlier steps left in the cache: portions of
prompts beside single decoded tokens, cut anywhere.  Everything above (scheduler, generation,
trace replay) goes through it.  The reference's counterpart is `RustDecoder::forward`
(rust/engine/src/rust_decoder.rs:8378-8398; batch validation :8551-8578; how the runtime builds
a batch: rust/engine/src/runtime.rs:2380-2442).
"""
from __future__ import annotations

import gc
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Union

import torch

from ..cache import CacheManager, OutOfPages
from ..config.files import read_config_json
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


# Decode steps are padded to these row counts and replayed as HIP graphs (the reference's
# buckets: rust/engine/src/rust_decoder.rs:1037; 80, 96 and 112 are this engine's own, where the feed-forward's kernels
# take five, six or seven row tiles instead of eight: a step of 96 requests 8.7 -> 7.9 ms at the 8B sizes).
GRAPH_BUCKETS = (1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64, 80, 96, 112, 128, 256)


class StepError(ValueError):
    """A batch the step function refuses before anything is launched."""


@dataclass
class StepEntry:
    """A request's next tokens.  `want`: indices into `tokens` whose logits are returned.
    `carry`: for an entry of one token that an earlier step chose and that is still on the
    device, its row in that step's token tensor (`tokens[0]` is then a placeholder)."""
    req_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()
    carry: Optional[int] = None


class ModelRunner:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype="bfloat16", device="cuda:0",
                 page_size: int = 16, max_tokens: Optional[int] = None,
                 num_pages: Union[int, Sequence[int], None] = None,
                 max_requests: int = 16, max_context: Optional[int] = None, memory_utilization: float = 0.90,
                 ops=None, typed_config=None, use_graphs: bool = True, max_step_tokens: Optional[int] = None,
                 decode_weight_tiles="auto", consume_tensors: bool = False):
        """`num_pages`: pages of every cache group (one number) or of each group (a list); by default what
        `max_tokens` tokens need, else what fits on the card.  `max_step_tokens`: the most tokens of one request
        that a step may bring (more are refused); with it, groups that keep a window of keys are made no larger than
        `max_requests` requests can fill.  `decode_weight_tiles`: True, False or "auto" (while memory is plentiful): the
        matrices whose products add into the residual stream keep a second, tile-major copy for decode steps
        (`Runtime.tile_for_decode`).  `consume_tensors`: the caller has no further use for `tensors`; the dictionary is
        emptied once the parts hold what they need, so that pieces the parts have joined into one matrix (q, k and v;
        gate and up) do not stay on the device beside it while the copies and the cache are sized."""
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
        self.rt = Runtime(self.device, self.dtype, ops, self.max_context, decode_weight_tiles)
        check_tensors(spec, {n: tuple(t.shape) for n, t in tensors.items()})
        self.model = Model(spec, tensors, self.rt, consume_tensors=consume_tensors)
        self.vocab_size = spec.vocab_size
        num_groups = len(self.model.group_keys)
        self.max_requests = max_requests
        self.max_step_tokens = None if max_step_tokens is None else int(max_step_tokens)
        if num_pages is None and max_tokens is not None:
            num_pages = -(-int(max_tokens) // page_size)
        if num_pages is None:
            pages = self._pages_that_fit(memory_utilization, max_requests)
        elif isinstance(num_pages, int):
            pages = [min(num_pages, cap) for cap in self._page_caps(max_requests)]
        else:
            pages = [int(n) for n in num_pages]
            if len(pages) != num_groups:
                raise ValueError(f"the model has {num_groups} cache groups, {len(pages)} page counts were given")
        if any(n <= 0 for n in pages):
            raise ValueError("the cache needs at least one page")
        self.pages_per_group = pages
        self.cache: CacheManager = self.model.allocate_caches(page_size, pages, max_requests,
                                                              max_step_tokens=self.max_step_tokens)
        self.steps = 0
        self.rows_total = 0
        # decode steps replay captured graphs when every part can be captured (parts say so with
        # `graph_safe`; a part that decides on the host per step cannot)
        parts_ok = all(getattr(b.mixer, "graph_safe", False)
                       and (b.feed_forward is None or getattr(b.feed_forward, "graph_safe", False))
                       and all(getattr(p, "graph_safe", False) for p in getattr(b, "extras", {}).values())
                       for b in self.model.blocks)
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and parts_ok
        self._graphs: Dict[tuple, "_DecodeGraph"] = {}
        self._graph_pool = None
        self.graph_replays = 0

    # ---- construction ---------------------------------------------------------------------
    @staticmethod
    def from_folder(model_dir: str, **kwargs) -> "ModelRunner":
        """The model class is chosen by config.json; weights are bound by tensor name."""
        config = read_config_json(model_dir)
        typed, spec = model_spec_from_config(config)
        tensors = load_checkpoint(model_dir, spec)
        return ModelRunner(spec, tensors, typed_config=typed, **kwargs)

    def _page_caps(self, max_requests: int) -> List[int]:
        """Per cache group the most pages `max_requests` requests can hold: whole contexts, or, for a group that
        keeps a window when steps are bounded, the window and one step."""
        caps = []
        for key in self.model.group_keys:
            window = key.window
            each = -(-self.max_context // self.page_size)
            if window is not None and self.max_step_tokens is not None:
                each = min(each, CacheManager.window_pages_bound(window, self.page_size, self.max_step_tokens))
            caps.append(max_requests * each)
        return caps

    def _pages_that_fit(self, utilization: float, max_requests: int) -> List[int]:
        """Pages for what is left of the card after the weights: window groups get what `max_requests` requests
        can fill, the other groups share the rest equally (a token needs a page of each), capped likewise."""
        per_page = self.model.cache_bytes_per_page(self.page_size)
        caps = self._page_caps(max_requests)
        if self.device.type != "cuda":
            return caps
        free, total = torch.cuda.mem_get_info(self.device)
        budget = int(free - (1.0 - utilization) * total) - (2 << 30)   # room for activations and logits
        bounded = [key.window is not None and self.max_step_tokens is not None for key in self.model.group_keys]
        pages = [cap if b else 0 for cap, b in zip(caps, bounded)]
        budget -= sum(n * size for n, size in zip(pages, per_page))
        rest = [g for g, b in enumerate(bounded) if not b]
        if rest:
            each = budget // max(1, sum(per_page[g] for g in rest))
            for g in rest:
                pages[g] = max(1, min(caps[g], each))
        return pages

    def check_layers(self, steps: int = 2, limit: float = 5e-2, out=None):
        """Switches the layer-by-layer check on for the next `steps` steps (see `diagnostics.LayerCheck`) and returns
        the object that collects the reports."""
        from .diagnostics import LayerCheck
        self.model.layer_check = LayerCheck(steps, limit, out)
        return self.model.layer_check

    # ---- requests -------------------------------------------------------------------------
    def add_request(self, req_id) -> int:
        return self.cache.add_request(req_id)

    def free_request(self, req_id) -> None:
        self.cache.free_request(req_id)

    def length(self, req_id) -> int:
        return self.cache.length(req_id)

    # ---- the step -------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry], previous_tokens: Optional[torch.Tensor] = None) -> None:
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
            if e.carry is not None:
                if n != 1:
                    raise StepError(f"request {e.req_id!r}: only an entry of one token can take it from an earlier step")
                if previous_tokens is None or not 0 <= int(e.carry) < previous_tokens.numel():
                    raise StepError(f"request {e.req_id!r} takes row {e.carry} of an earlier step's tokens, which has "
                                    f"{0 if previous_tokens is None else previous_tokens.numel()}")
            for t in (e.tokens if e.carry is None else ()):
                if not 0 <= int(t) < self.vocab_size:
                    raise StepError(f"token id {t} of request {e.req_id!r} is outside [0, {self.vocab_size})")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.req_id!r} wants logits at {w}, it brings {n} tokens")
            if self.max_step_tokens is not None and n > self.max_step_tokens:
                raise StepError(f"request {e.req_id!r} brings {n} tokens, a step takes at most {self.max_step_tokens} of a request")
            start = self.cache.length(e.req_id) if self.cache.has_request(e.req_id) else 0
            if start + n > self.max_context:
                raise StepError(f"request {e.req_id!r} would hold {start + n} tokens, the context is {self.max_context}")
            multiple = self.model.portion_multiple
            if multiple > 1 and n > 1 and start % multiple != 0:
                raise StepError(f"request {e.req_id!r} brings a portion of {n} tokens at position {start}: portions of this "
                                f"model begin on multiples of {multiple}")

    # ---- per-request state of fixed size ----------------------------------------------------
    def snapshot_state(self, req_id):
        """A copy of everything the model's layers keep for `req_id` outside the pages, as it is after the steps
        launched so far (the reference's rust/engine/src/rust_decoder/state_api.rs:84-120); [] for a model without."""
        return self.model.snapshot_state(self.cache.slot(req_id))

    def restore_state(self, req_id, snapshot) -> None:
        """Puts a snapshot of this model into the slot of `req_id` (a request that the cache manager knows: its length
        says how many tokens the state stands for, state_api.rs:122-160).  The next step of the request goes on there."""
        self.model.restore_state(self.cache.slot(req_id), snapshot)

    def step(self, entries: Sequence[StepEntry], previous_tokens: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs the entries as one batch and returns float32 logits [wanted, vocab] on the device,
        in the order of the entries and of each entry's `want`; they are valid until the next step (decode steps
        replay graphs that write them in place).  Unknown requests are added.
        Raises `OutOfPages` (nothing changed) when the pages do not suffice.
        `previous_tokens`: the int32 device tensor that entries with `carry` take their token from."""
        self._validate(entries, previous_tokens)
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
        if self.model.has_state:
            for e in entries:                # a request's first step finds its state slot cleared
                if self.cache.length(e.req_id) == 0:
                    self.model.clear_state(self.cache.slot(e.req_id))
        logits = None
        checking = self.model.layer_check is not None and self.model.layer_check.active     # checked steps run eagerly
        if not checking and self.use_graphs and all(len(e.tokens) == 1 for e in entries) and len(entries) <= GRAPH_BUCKETS[-1]:
            logits = self._graph_step(entries, previous_tokens)
        if logits is None:
            ctx = self._build_context(entries, previous_tokens)
            logits = self.model.forward(ctx)
        for e in entries:
            self.cache.commit(e.req_id, len(e.tokens))
        self.steps += 1
        self.rows_total += sum(len(e.tokens) for e in entries)
        return logits

    # ---- decode steps as HIP graphs ---------------------------------------------------------
    def _graph_step(self, entries: Sequence[StepEntry], previous_tokens: Optional[torch.Tensor] = None
                    ) -> Optional[torch.Tensor]:
        """A step of single-token entries, padded to a bucket and replayed as a graph.  The graph is
        captured at the first use of a (rows, context bound) pair, after one eager run of the same
        shape.  Padding rows belong to no segment (row_seg -1): they store nothing and their output
        is dropped."""
        import numpy as np
        count = len(entries)
        bucket = next(b for b in GRAPH_BUCKETS if b >= count)
        starts = [self.cache.length(e.req_id) for e in entries]
        bound = 256
        while bound < max(starts) + 1:
            bound *= 2
        bound = min(bound, self.max_context)
        widths = [-(-bound // g.page_size) for g in self.cache.groups]
        key = (bucket, bound)
        graph = self._graphs.get(key)
        if graph is None:
            graph = _DecodeGraph(self, bucket, bound, widths)
            self._graphs[key] = graph
        graph.done.synchronize()                  # the previous copy out of the pinned buffer has finished
        h = graph.host_np
        h[:] = graph.template
        B = bucket
        h[0:count] = [int(e.tokens[0]) if e.carry is None else 0 for e in entries]
        h[B:B + count] = starts
        h[2 * B:2 * B + count] = np.arange(count)
        h[4 * B + 1:4 * B + 1 + count] = [self.cache.slot(e.req_id) for e in entries]
        o = 6 * B + 1
        for g, width in enumerate(widths):
            tables = h[o:o + B * width].reshape(B, width)
            for i, e in enumerate(entries):
                # a table may be longer than the graph's rows (pages reserved ahead, for the rest of a prompt or by
                # the caller): the row at position `start` reads entries up to start / page_size, all below `width`
                t = self.cache.table(e.req_id, g)[:width]
                tables[i, :len(t)] = t
            o += B * width
        carried = any(e.carry is not None for e in entries)
        if carried:
            h[graph.carry_at:graph.carry_at + count] = [-1 if e.carry is None else int(e.carry) for e in entries]
        graph.device_buf.copy_(graph.host_buf, non_blocking=True)
        graph.done.record()
        if carried:
            self.rt.ops.carry_ids(graph.ctx.ids, graph.carry_source, previous_tokens)
        if graph.graph is None:
            graph.capture()
        graph.graph.replay()
        self.graph_replays += 1
        wanted = [i for i, e in enumerate(entries) if len(e.want)]
        if len(wanted) == bucket:
            return graph.logits
        if len(wanted) == count and count > 0 and wanted == list(range(count)):
            return graph.logits[:count]
        index = torch.tensor(wanted, dtype=torch.long, device=self.device)
        return graph.logits.index_select(0, index)

    def capture_graphs(self, row_counts: Sequence[int], context_bounds: Sequence[int]) -> int:
        """Captures the decode graphs of these (rows, context bound) pairs before a step needs them (rows are rounded up
        to buckets, bounds to the powers of two from 256 that graphs are keyed by).  Every row of such a capture is a
        padding row: nothing is stored.  Returns the number of graphs captured."""
        if not self.use_graphs:
            return 0
        made = 0
        buckets = sorted({next(b for b in GRAPH_BUCKETS if b >= min(n, GRAPH_BUCKETS[-1])) for n in row_counts if n > 0})
        bounds = set()
        for limit in context_bounds:
            bound = 256
            while bound < limit:
                bound *= 2
            bounds.add(min(bound, self.max_context))
        for bucket in buckets:
            for bound in sorted(bounds):
                if (bucket, bound) in self._graphs:
                    continue
                widths = [-(-bound // g.page_size) for g in self.cache.groups]
                graph = _DecodeGraph(self, bucket, bound, widths)
                graph.host_np[:] = graph.template
                graph.device_buf.copy_(graph.host_buf, non_blocking=True)
                graph.done.record()
                graph.capture()
                self._graphs[(bucket, bound)] = graph
                made += 1
        return made

    def _build_context(self, entries: Sequence[StepEntry], previous_tokens: Optional[torch.Tensor] = None) -> StepContext:
        ids: List[int] = []
        row_pos: List[int] = []
        row_seg: List[int] = []
        slots: List[int] = []
        logit_rows: List[int] = []
        seg_rows, seg_start = [], []
        carry: Dict[int, int] = {}              # row -> row of the earlier step's tokens
        max_context = 0
        # Segments of several rows first, single rows behind them (attention treats the two kinds differently); the
        # logits keep the order of the caller's entries.
        order = sorted(range(len(entries)), key=lambda i: len(entries[i].tokens) == 1)
        base_of = {}
        for s, i in enumerate(order):
            e = entries[i]
            start = self.cache.length(e.req_id)
            n = len(e.tokens)
            base = base_of[i] = len(ids)
            if e.carry is not None:
                carry[base] = int(e.carry)
                ids.append(0)
            else:
                ids.extend(int(t) for t in e.tokens)
            row_pos.extend(range(start, start + n))
            row_seg.extend([s] * n)
            slots.append(self.cache.slot(e.req_id))
            seg_rows.append(n)
            seg_start.append(start)
            max_context = max(max_context, start + n)
        for i, e in enumerate(entries):
            logit_rows.extend(base_of[i] + int(w) for w in e.want)
        single_from = sum(1 for n in seg_rows if n != 1)
        single_max_context = max((start + 1 for start, n in zip(seg_start, seg_rows) if n == 1), default=0)
        entries = [entries[i] for i in order]       # the tables below follow the segments
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
        R, L = len(ids), len(logit_rows)
        source = [carry.get(r, -1) for r in range(R)] if carry else []
        packed = torch.tensor(ids + row_pos + row_seg + cu_rows + slots + logit_rows + flat_tables + source, dtype=torch.int32)
        if self.device.type == "cuda":   # from pinned memory, so that the copy does not wait for the step before
            packed = packed.pin_memory().to(self.device, non_blocking=True)
        else:
            packed = packed.to(self.device)
        o = 0

        def take(count):
            nonlocal o
            out = packed[o:o + count]
            o += count
            return out

        t_ids, t_pos, t_seg, t_cu, t_slots, t_rows = take(R), take(R), take(R), take(S + 1), take(S), take(L)
        tables = [take(S * w).view(S, w) for w in widths]
        if carry:
            self.rt.ops.carry_ids(t_ids, take(R), previous_tokens)
        return StepContext(num_rows=R, num_segments=S, ids=t_ids, row_pos=t_pos, row_seg=t_seg, seg_start=t_cu,
                           slots=t_slots,
                           logit_rows=t_rows, tables=tables, seg_rows=seg_rows, seg_pos_start=seg_start,
                           seg_slots=slots, max_context=max_context, uniform_rows=all(n == 1 for n in seg_rows),
                           single_from=single_from, single_max_context=single_max_context)


class _DecodeGraph:
    """Static buffers and the captured graph of decode steps of `bucket` rows whose contexts stay
    within `bound` tokens.  Buffer layout (int32): ids[B], row_pos[B], row_seg[B], seg_start[B+1],
    slots[B], logit_rows[B], then per cache group tables[B, width]."""

    def __init__(self, runner: "ModelRunner", bucket: int, bound: int, widths):
        import numpy as np
        self.runner = runner
        self.bucket = bucket
        self.bound = bound
        B = bucket
        self.carry_at = 6 * B + 1 + sum(B * w for w in widths)     # behind the tables: where each row's token comes from
        size = self.carry_at + B
        self.host_buf = torch.zeros(size, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host_buf.numpy()
        template = np.zeros(size, dtype=np.int32)
        template[2 * B:3 * B] = -1                              # row_seg of padding rows
        template[3 * B:4 * B + 1] = np.arange(B + 1)            # one row per segment
        template[5 * B + 1:6 * B + 1] = np.arange(B)            # logits of every row
        template[self.carry_at:self.carry_at + B] = -1          # tokens come from the host
        self.template = template
        self.device_buf = torch.zeros(size, dtype=torch.int32, device=runner.device)
        self.done = torch.cuda.Event()
        self.done.record()
        d = self.device_buf
        o = 6 * B + 1
        tables = []
        for w in widths:
            tables.append(d[o:o + B * w].view(B, w))
            o += B * w
        self.ctx = StepContext(num_rows=B, num_segments=B, ids=d[0:B], row_pos=d[B:2 * B], row_seg=d[2 * B:3 * B],
                               seg_start=d[3 * B:4 * B + 1], slots=d[4 * B + 1:5 * B + 1],
                               logit_rows=d[5 * B + 1:6 * B + 1], tables=tables, seg_rows=[1] * B,
                               seg_pos_start=[0] * B, seg_slots=[0] * B, max_context=bound, uniform_rows=True)
        self.carry_source = d[self.carry_at:self.carry_at + B]
        self.graph = None
        self.logits = None

    def capture(self) -> None:
        runner = self.runner
        runner.model.forward(self.ctx)                  # eager once: every kernel of this shape has run before capture
        torch.cuda.synchronize(runner.device)
        if runner._graph_pool is None:
            runner._graph_pool = torch.cuda.graph_pool_handle()
        graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: a collector that frees what an engine before this
        # one left behind (its graphs, its pinned buffers) calls into the HIP runtime, which refuses such calls
        # during a capture, and a failure inside a destructor ends the process.
        collecting = gc.isenabled()
        gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=runner._graph_pool):
                self.logits = runner.model.forward(self.ctx)
        finally:
            if collecting:
                gc.enable()
        self.graph = graph
