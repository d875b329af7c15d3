"""Cache manager: which pages hold which tokens of which request, for every group of layers,
and a slot of fixed-size state per live request.

A *group* is a set of cache-owning run entries with the same need: all keys, or a window of
them.  Each group has a page pool and per-request block tables of its own
(rust/engine/src/mem/block_allocator.rs:146-312 `BlockManager`, :317-376 `HybridBlockManager`).
Table entry i of a request covers positions [i * page_size, (i + 1) * page_size); an entry is
-1 once a window has passed the page and it was given back (:286-311 `prune_sliding_window`).

Lifecycle of a request: `add_request` (takes a state slot), then per step `reserve(total)`
before the step (pages for every position below `total`; fails without changing anything,
block_allocator.rs:231-253) and `commit(n)` after it (the request now holds n more tokens;
pages behind a window go back), finally `free_request` (all pages and the slot go back).
This module is bookkeeping only: it never touches device memory.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence

from .pages import OutOfPages, PagePool


@dataclass(frozen=True)
class GroupSpec:
    """Cache-owning run entries with one need.  `window` None: all keys are kept."""
    entries: tuple
    kv_heads: int
    head_dim: int
    window: Optional[int]
    page_size: int


@dataclass
class _Request:
    slot: int
    length: int = 0                                   # committed tokens
    tables: List[List[int]] = field(default_factory=list)   # per group


class CacheManager:
    def __init__(self, groups: Sequence[GroupSpec], pages_per_group: Sequence[int], max_requests: int,
                 max_step_tokens: Optional[int] = None):
        """`max_step_tokens`: the most tokens of one request that a step brings, when the caller keeps to such a
        bound.  A window group then never holds pages further ahead of a request than one step can reach, however
        far a reservation looks (a whole prompt at admission): its pool can be made for
        `window_pages_bound` pages a request instead of a whole context."""
        if len(groups) != len(pages_per_group):
            raise ValueError("one page count per group is required")
        if max_requests <= 0:
            raise ValueError("max_requests must be positive")
        if max_step_tokens is not None and max_step_tokens <= 0:
            raise ValueError("max_step_tokens must be positive")
        self.max_step_tokens = max_step_tokens
        self.groups = list(groups)
        self.pools = [PagePool(n) for n in pages_per_group]
        self.max_requests = max_requests
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self._requests: Dict[object, _Request] = {}

    # ---- requests -------------------------------------------------------------------------
    def add_request(self, req_id) -> int:
        if req_id in self._requests:
            raise ValueError(f"request {req_id!r} already holds a cache")
        if not self._free_slots:
            raise OutOfPages(f"all {self.max_requests} request slots are taken")
        slot = self._free_slots.pop()
        self._requests[req_id] = _Request(slot=slot, tables=[[] for _ in self.groups])
        return slot

    def has_request(self, req_id) -> bool:
        return req_id in self._requests

    def requests(self):
        return list(self._requests)

    def free_request(self, req_id) -> None:
        req = self._requests.pop(req_id, None)
        if req is None:
            return
        for g, table in enumerate(req.tables):
            for page in table:
                if page >= 0:
                    self.pools[g].release(page)
        self._free_slots.append(req.slot)

    def _get(self, req_id) -> _Request:
        try:
            return self._requests[req_id]
        except KeyError:
            raise KeyError(f"request {req_id!r} holds no cache") from None

    def slot(self, req_id) -> int:
        return self._get(req_id).slot

    def length(self, req_id) -> int:
        return self._get(req_id).length

    def table(self, req_id, group: int) -> List[int]:
        return self._get(req_id).tables[group]

    def free_slots(self) -> int:
        return len(self._free_slots)

    def free_pages(self, group: int = 0) -> int:
        return self.pools[group].available

    # ---- pages ----------------------------------------------------------------------------
    def _first_needed_page(self, group: GroupSpec, length: int) -> int:
        """First table index a request of committed `length` may still read: the next row sits at
        position >= length and sees keys from length - window + 1 on."""
        if group.window is None:
            return 0
        return max(0, length - group.window + 1) // group.page_size

    def _covered_upto(self, group: GroupSpec, length: int, total: int) -> int:
        """Table entries below this index are to hold pages so that positions below `total` are covered; in a window
        group no further than the next step can reach."""
        if group.window is not None and self.max_step_tokens is not None:
            total = min(total, length + self.max_step_tokens)
        return -(-total // group.page_size)

    @staticmethod
    def window_pages_bound(window: int, page_size: int, max_step_tokens: int) -> int:
        """Most pages a request holds in a window group when no step brings more than `max_step_tokens` of its
        tokens: the window before the step's first row, the step's rows, and the page edges on both sides."""
        return -(-(window - 1 + max_step_tokens) // page_size) + 1

    def pages_missing(self, req_id, total: int) -> List[int]:
        """Pages each group would have to hand out so that positions below `total` are covered.
        Every table entry from the first page still needed to the end of the table holds a page
        (`reserve` fills them, `commit` takes pages away only below that point, `trim` only at the
        end), so what is missing is the stretch behind the table."""
        req = self._get(req_id)
        out = []
        for g, group in enumerate(self.groups):
            need_upto = self._covered_upto(group, req.length, total)
            have_upto = max(len(req.tables[g]), self._first_needed_page(group, req.length))
            out.append(max(0, need_upto - have_upto))
        return out

    def can_reserve(self, req_id, total: int) -> bool:
        return all(m <= pool.available for m, pool in zip(self.pages_missing(req_id, total), self.pools))

    def reserve(self, req_id, total: int) -> None:
        """Covers positions below `total` in every group, or raises `OutOfPages` and changes nothing."""
        missing = self.pages_missing(req_id, total)
        for g, (m, pool) in enumerate(zip(missing, self.pools)):
            if m > pool.available:
                raise OutOfPages(f"group {g} needs {m} pages, {pool.available} are free")
        req = self._get(req_id)
        for g, group in enumerate(self.groups):
            need_upto = self._covered_upto(group, req.length, total)
            table = req.tables[g]
            first = self._first_needed_page(group, req.length)
            start = max(first, len(table))          # entries below `first` are never read again: they stay empty
            while len(table) < need_upto:
                table.append(-1)
            for i in range(start, need_upto):
                table[i] = self.pools[g].alloc()

    def commit(self, req_id, count: int) -> None:
        """The request holds `count` more tokens; pages a window has passed go back."""
        if count < 0:
            raise ValueError("count must be nonnegative")
        req = self._get(req_id)
        new_length = req.length + count
        for g, group in enumerate(self.groups):
            if -(-new_length // group.page_size) > len(req.tables[g]):
                raise ValueError(f"request {req_id!r} commits {new_length} tokens but holds pages for fewer")
        req.length = new_length
        for g, group in enumerate(self.groups):
            if group.window is None:
                continue
            table = req.tables[g]
            for i in range(min(self._first_needed_page(group, new_length), len(table))):
                if table[i] >= 0:
                    self.pools[g].release(table[i])
                    table[i] = -1

    def trim(self, req_id, total: int) -> None:
        """Gives back pages that cover nothing below `total` (a reservation that was not used)."""
        req = self._get(req_id)
        if total < req.length:
            raise ValueError("cannot trim below the committed length")
        for g, group in enumerate(self.groups):
            keep = -(-total // group.page_size)
            table = req.tables[g]
            while len(table) > keep:
                page = table.pop()
                if page >= 0:
                    self.pools[g].release(page)

    # ---- self check -----------------------------------------------------------------------
    def check_invariants(self) -> None:
        """No page lost, none held twice, none both free and held; slots likewise."""
        for g, pool in enumerate(self.pools):
            held: Dict[int, int] = {}
            for req in self._requests.values():
                for page in req.tables[g]:
                    if page >= 0:
                        held[page] = held.get(page, 0) + 1
            free = list(pool._free)
            if len(set(free)) != len(free):
                raise AssertionError(f"group {g}: a page is on the free list twice")
            for page in range(pool.num_pages):
                if pool.refcounts[page] != held.get(page, 0):
                    raise AssertionError(f"group {g}: page {page} has refcount {pool.refcounts[page]}, "
                                         f"tables hold it {held.get(page, 0)} times")
                if (pool.refcounts[page] == 0) != (page in set(free)):
                    raise AssertionError(f"group {g}: page {page} is neither free nor held, or both")
        for req_id, req in self._requests.items():
            for g, group in enumerate(self.groups):
                first = self._first_needed_page(group, req.length)
                if any(page < 0 for page in req.tables[g][first:]):
                    raise AssertionError(f"group {g}: request {req_id!r} misses a page it may still read")
        slots = [r.slot for r in self._requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_slots):
            raise AssertionError("a state slot is held twice")
        if len(slots) + len(self._free_slots) != self.max_requests:
            raise AssertionError("a state slot was lost")
