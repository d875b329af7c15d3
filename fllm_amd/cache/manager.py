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
from .prefix import PrefixIndex, PrefixNode


@dataclass(frozen=True)
class GroupSpec:
    """Cache-owning run entries with one need.  `window` None: all keys are kept."""
    entries: tuple
    kv_heads: int
    k_dim: int
    v_dim: int
    window: Optional[int]
    page_size: int


@dataclass
class _Request:
    slot: int
    length: int = 0                                   # committed tokens
    tables: List[List[int]] = field(default_factory=list)   # per group
    shared: List[PrefixNode] = field(default_factory=list)  # the prefix index's nodes for this request's first pages, in order


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
        self.prefix: Optional[PrefixIndex] = None
        # nodes of the index that no live request holds, in the order in which they may be given up: the one unused
        # for longest first, and the pages behind a node always before the node itself
        self._idle: Dict[PrefixNode, None] = {}
        self.prefix_hit_tokens = 0

    # ---- prefixes shared between requests ---------------------------------------------------
    def enable_prefix_cache(self) -> None:
        """From now on full pages stay after their request has ended and serve later requests that begin with the
        same tokens, until the room is needed.  Only where every group keeps all keys with one page size: a window
        gives pages back that a later request would need, and a prefix is counted in pages."""
        if any(g.window is not None for g in self.groups) or len({g.page_size for g in self.groups}) != 1:
            raise ValueError("the prefix cache needs cache groups that keep all keys, with one page size")
        if self.prefix is None:
            self.prefix = PrefixIndex(self.groups[0].page_size)

    def _hold(self, req: _Request, node: PrefixNode) -> None:
        node.holders += 1
        self._idle.pop(node, None)
        req.shared.append(node)

    def _known_prefix(self, tokens: Sequence[int], with_state: bool) -> List[PrefixNode]:
        """The nodes of the longest known prefix of `tokens` that leaves at least the last token to be computed; where
        the model keeps state per request (`with_state`), only as far as a node that holds a copy of that state."""
        if self.prefix is None:
            return []
        nodes = self.prefix.match(tokens, (len(tokens) - 1) // self.prefix.page_size)
        if with_state:
            while nodes and nodes[-1].state is None:
                nodes.pop()
        return nodes

    def probe_prefix(self, tokens: Sequence[int], with_state: bool = False):
        """(pages, idle) of what `adopt_prefix` would take over: how many pages, and how many of them no request holds
        at the moment (those count among `free_pages` until they are adopted).  Changes nothing."""
        nodes = self._known_prefix(tokens, with_state)
        return len(nodes), sum(1 for n in nodes if n.holders == 0)

    def adopt_prefix(self, req_id, tokens: Sequence[int], with_state: bool = False):
        """For a request that holds nothing yet: puts the pages of the longest known prefix of `tokens` into its block
        tables, leaving at least the last token to be computed.  Returns the number of tokens taken over; the request
        holds them as if it had committed them.  `with_state`: only as far as a page behind which a copy of the
        model's per-request state was kept (`keep_state`); then (tokens, that copy) is returned."""
        req = self._get(req_id)
        if self.prefix is None or req.length != 0 or any(req.tables):
            return (0, None) if with_state else 0
        page_size = self.prefix.page_size
        for node in self._known_prefix(tokens, with_state):
            for g, page in enumerate(node.pages):
                self.pools[g].retain(page)
                req.tables[g].append(page)
            self._hold(req, node)
        req.length = len(req.shared) * page_size
        self.prefix_hit_tokens += req.length
        if with_state:
            return req.length, (req.shared[-1].state if req.shared else None)
        return req.length

    def keep_state(self, req_id, tokens: int, state) -> bool:
        """Keeps `state` (whatever the caller copies a request's fixed-size state into) with the known prefix that ends
        behind the request's first `tokens` tokens, which must be whole pages that `remember_prefix` has entered.
        False: there is no such prefix (the prefix cache is off, or the page was not entered)."""
        req = self._get(req_id)
        if self.prefix is None or tokens <= 0 or tokens % self.prefix.page_size != 0:
            return False
        index = tokens // self.prefix.page_size - 1
        if index >= len(req.shared):
            return False
        if req.shared[index].state is None:
            req.shared[index].state = state
        return True

    def share_pages(self, src_id, dst_id, tokens: int) -> int:
        """For a request `dst_id` that holds nothing yet: puts the full pages of `src_id` that lie wholly below `tokens`
        (and below what `src_id` has committed) into its block tables as well, and counts them as committed.  The
        caller's word: both requests have the same tokens there.  Neither writes such a page again: each writes at and
        behind its committed length.  Returns the tokens shared; 0 where a group has a window (its pages go back
        while the request runs), where page sizes differ between groups, and with the prefix index on (which serves
        the same purpose through `adopt_prefix`)."""
        src, dst = self._get(src_id), self._get(dst_id)
        if dst.length != 0 or any(dst.tables) or self.prefix is not None:
            return 0
        if not self.groups:                     # a model without keys and values: nothing to share but the position
            dst.length = min(src.length, int(tokens))
            return dst.length
        if any(g.window is not None for g in self.groups) or len({g.page_size for g in self.groups}) != 1:
            return 0
        page_size = self.groups[0].page_size
        pages = min(src.length, int(tokens)) // page_size
        for g in range(len(self.groups)):
            for page in src.tables[g][:pages]:
                self.pools[g].retain(page)
                dst.tables[g].append(page)
        dst.length = pages * page_size
        return dst.length

    def remember_prefix(self, req_id, tokens: Sequence[int], known: Optional[int] = None) -> None:
        """Enters the full pages of a request into the index.  `tokens` are the request's tokens from its first on, of
        which the first `known` are final; pages wholly below that and below the committed length are entered.  Where
        another request has entered the same tokens meanwhile, this one goes on with that one's pages and gives its
        own back (same tokens at the same places: same keys and values)."""
        if self.prefix is None:
            return
        req = self._get(req_id)
        page_size = self.prefix.page_size
        full = min(len(tokens) if known is None else known, req.length) // page_size
        while len(req.shared) < full:
            i = len(req.shared)
            parent = req.shared[-1] if req.shared else None
            key = tuple(tokens[i * page_size:(i + 1) * page_size])
            node = self.prefix.child(parent, key)
            if node is None:
                pages = tuple(req.tables[g][i] for g in range(len(self.groups)))
                for g, page in enumerate(pages):
                    self.pools[g].retain(page)           # the index's own reference
                node = self.prefix.insert(parent, key, pages)
            else:
                for g, page in enumerate(node.pages):
                    if req.tables[g][i] != page:
                        self.pools[g].retain(page)
                        self.pools[g].release(req.tables[g][i])
                        req.tables[g][i] = page
            self._hold(req, node)

    def cached_pages(self) -> int:
        return self.prefix.size if self.prefix is not None else 0

    def clear_prefixes(self) -> int:
        """Gives up every known prefix that no request holds; returns how many pages a group got back."""
        dropped = len(self._idle)
        for g in range(len(self.groups)):
            self._make_room(g, self.pools[g].num_pages + 1)
        return dropped

    def _make_room(self, group: int, needed: int) -> None:
        """Gives up unused prefixes, the longest unused first and from their ends, until `needed` pages are free."""
        while self.pools[group].available < needed and self._idle:
            node = next(iter(self._idle))
            del self._idle[node]
            self.prefix.remove(node)
            for g, page in enumerate(node.pages):
                self.pools[g].release(page)

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
        for node in reversed(req.shared):               # the end of a prefix goes before its beginning
            node.holders -= 1
            if node.holders == 0:
                self._idle[node] = None
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
        """Pages that a reservation can get: the free ones and those of known prefixes that no request holds."""
        return self.pools[group].available + len(self._idle)

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
        return all(m <= self.free_pages(g) for g, m in enumerate(self.pages_missing(req_id, total)))

    def reserve(self, req_id, total: int) -> None:
        """Covers positions below `total` in every group, or raises `OutOfPages` and changes nothing."""
        missing = self.pages_missing(req_id, total)
        for g, m in enumerate(missing):
            if m > self.free_pages(g):
                raise OutOfPages(f"group {g} needs {m} pages, {self.free_pages(g)} are free")
        for g, m in enumerate(missing):
            self._make_room(g, m)
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
        """No page lost, none held twice, none both free and held; slots likewise.  With shared prefixes: every
        reference is a block table's or the index's, and the index agrees with the tables."""
        nodes = self.prefix.nodes() if self.prefix is not None else []
        holders: Dict[PrefixNode, int] = {}
        for req_id, req in self._requests.items():
            for i, node in enumerate(req.shared):
                holders[node] = holders.get(node, 0) + 1
                if node.parent is not (req.shared[i - 1] if i else self.prefix.root):
                    raise AssertionError(f"request {req_id!r}: its shared pages are no chain from the first page on")
                if any(req.tables[g][i] != page for g, page in enumerate(node.pages)):
                    raise AssertionError(f"request {req_id!r}: page {i} is shared but its table names another page")
            if len(req.shared) * (self.prefix.page_size if self.prefix else 0) > req.length:
                raise AssertionError(f"request {req_id!r} shares pages it has not committed")
        for node in nodes:
            if node.holders != holders.get(node, 0):
                raise AssertionError(f"a prefix node counts {node.holders} holders, {holders.get(node, 0)} requests hold it")
            if (node.holders == 0) != (node in self._idle):
                raise AssertionError("a prefix node is unused and not up for reuse, or the other way round")
        if len(self._idle) != sum(1 for node in nodes if node.holders == 0):
            raise AssertionError("a node that is up for reuse is not in the index")
        seen_idle = set()
        for node in self._idle:
            if any(child not in seen_idle for child in node.children.values()):
                raise AssertionError("a prefix would be given up before what lies behind it")
            seen_idle.add(node)
        for g, pool in enumerate(self.pools):
            held: Dict[int, int] = {}
            for node in nodes:
                held[node.pages[g]] = held.get(node.pages[g], 0) + 1
                if held[node.pages[g]] > 1:
                    raise AssertionError(f"group {g}: page {node.pages[g]} stands for two prefixes")
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
