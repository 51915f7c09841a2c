"""The cache manager: which request holds which pages of which group, and which state slot.

Runs of layers with the same needs (key/value heads, head size, all keys or a window of them) form a
*group*.  Every group has a pool of pages and an allocator of its own, and every request has one block
table per group: entry i is the page holding its keys i*page_size .. (i+1)*page_size-1 in every run of
the group.  A windowed group gives pages back as soon as the window has passed them (their table entry
becomes the null page); everything is given back when the request ends.  Beside the pages each request
holds one *row* from admission to its end: the row indexes the block tables and is the request's slot in
the fixed-size state tensors of the runs that keep such state.

Only bookkeeping lives here (lists and numpy tables); the device memory is in ``pools.py``.
The reference keeps one table per request shared by all layers (src/miniserve/engine.py:57,
paged.py:188-194), allocates ceil(P / block_size) pages for a prompt up front and one page when a decoded
token starts a new one (paged_engine.py:115-121, 152-155), and frees on finish, preemption and cancel
(paged_engine.py:179-196).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence, Tuple

import numpy as np

from .allocator import NULL_PAGE, OutOfPages, PageAllocator


@dataclass(frozen=True)
class GroupKey:
    """What the pages of a group hold (a tuple of ``parts.base.PageTensor``) and for how long."""

    tensors: tuple
    window: Optional[int]

    def values_per_token(self) -> int:
        return sum(t.heads * t.width for t in self.tensors)


@dataclass
class CacheGroup:
    key: GroupKey
    runs: List[int]                 # runs of the model's order that keep their cache here
    allocator: PageAllocator
    tables: np.ndarray              # int32 [max_requests, max_pages_per_request]


@dataclass
class _Held:
    row: int
    computed: int = 0                                   # tokens whose keys/values (and state) are stored
    next_page: List[int] = field(default_factory=list)  # per group: logical pages allocated so far
    first_live: List[int] = field(default_factory=list)  # per group: first logical page not yet given back


class CacheLayout:
    """How the runs of a model map to groups and state tensors (derived from ``Model.run_needs()``)."""

    def __init__(self, run_needs: Sequence[Tuple[object, object, Optional[int]]]):
        self.group_keys: List[GroupKey] = []
        self.group_runs: List[List[int]] = []
        self.run_group: List[Optional[int]] = []   # group of each run's own or borrowed cache
        self.run_entry: List[Optional[int]] = []   # index of the run's pages inside its group
        self.run_stores: List[bool] = []
        self.state_runs: List[int] = []
        self.state_needs: Dict[int, object] = {}
        for i, (kv, state, cache_of) in enumerate(run_needs):
            if cache_of is not None:
                if kv is None:
                    raise ValueError(f"run {i} reads the cache of run {cache_of} but its mixer keeps no keys and values")
                src_kv = run_needs[cache_of][0]
                if src_kv is None or src_kv.tensors != kv.tensors:
                    raise ValueError(f"run {i} cannot read the cache of run {cache_of}: their pages hold different tensors")
                if src_kv.window is not None and (kv.window is None or kv.window > src_kv.window):
                    raise ValueError(f"run {i} looks further back than run {cache_of}, whose cache it reads, keeps keys")
                self.run_group.append(self.run_group[cache_of])
                self.run_entry.append(self.run_entry[cache_of])
                self.run_stores.append(False)
            elif kv is not None:
                key = GroupKey(tuple(kv.tensors), kv.window)
                if key not in self.group_keys:
                    self.group_keys.append(key)
                    self.group_runs.append([])
                g = self.group_keys.index(key)
                self.run_group.append(g)
                self.run_entry.append(len(self.group_runs[g]))
                self.group_runs[g].append(i)
                self.run_stores.append(True)
            else:
                self.run_group.append(None)
                self.run_entry.append(None)
                self.run_stores.append(False)
            if state is not None:
                self.state_runs.append(i)
                self.state_needs[i] = tuple(state) if isinstance(state, (tuple, list)) else state


    def bytes_per_token(self, bytes_per_value: int) -> int:
        """Stored bytes per token over all runs that keep a cache (for keys and values: layers x 2 x kv heads
        x head size x bytes, src/miniserve/cache.py:27-29)."""
        return sum(len(runs) * key.values_per_token() * bytes_per_value
                   for key, runs in zip(self.group_keys, self.group_runs))


class CacheManager:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages, max_requests: int, max_len: int):
        """``num_pages`` usable pages in every group's pool, or one number per group (a group that keeps a tenth
        of the bytes per token may be given a pool of its own size); a request may hold up to ``max_len`` tokens.
        The block tables have one row per request and a last row that stays all null pages (rows that pad a
        captured batch read it)."""
        if page_size <= 0 or max_requests <= 0 or max_len <= 0:
            raise ValueError("page_size, max_requests and max_len must be positive")
        self.layout = layout
        n_groups = len(layout.group_keys)
        per_group = [int(num_pages)] * n_groups if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if len(per_group) != n_groups:
            raise ValueError(f"{len(per_group)} pool sizes for {n_groups} cache groups")
        self.page_size, self.pages_per_group = page_size, per_group
        self.num_pages = min(per_group) if per_group else int(num_pages if isinstance(num_pages, int) else 0)
        self.max_requests, self.max_len = max_requests, max_len
        self.max_pages_per_request = -(-max_len // page_size)
        self.null_row = max_requests
        self.groups: List[CacheGroup] = [
            CacheGroup(key, runs, PageAllocator(n),
                       np.zeros((max_requests + 1, self.max_pages_per_request), dtype=np.int32))
            for key, runs, n in zip(layout.group_keys, layout.group_runs, per_group)]
        self._free_rows = list(range(max_requests - 1, -1, -1))
        self._held: Dict[Hashable, _Held] = {}
        # table entries that changed since ``take_updates`` was last called, per group: flat index -> page
        self._changed: List[Dict[int, int]] = [{} for _ in self.groups]

    # ------------------------------------------------------------------ requests
    def has(self, req_id) -> bool:
        return req_id in self._held

    def num_requests(self) -> int:
        return len(self._held)

    def free_rows(self) -> int:
        return len(self._free_rows)

    def add(self, req_id) -> int:
        """Give the request a row (its state slot).  It holds no pages yet."""
        if req_id in self._held:
            raise ValueError(f"request {req_id!r} is already held")
        if not self._free_rows:
            raise OutOfPages(f"all {self.max_requests} request rows are taken")
        row = self._free_rows.pop()
        n = len(self.groups)
        self._held[req_id] = _Held(row, 0, [0] * n, [0] * n)
        return row

    def row(self, req_id) -> int:
        return self._held[req_id].row

    def computed(self, req_id) -> int:
        return self._held[req_id].computed

    def capacity_tokens(self) -> int:
        """Tokens one request could hold if it had the smallest pool to itself."""
        return min(self.max_len, self.num_pages * self.page_size) if self.groups else self.max_len

    # ------------------------------------------------------------------ pages
    def _first_needed(self, g: CacheGroup, computed: int) -> int:
        """First logical page a query at position >= ``computed`` can still see."""
        if g.key.window is None:
            return 0
        return max(0, computed - g.key.window + 1) // self.page_size

    def _set(self, gi: int, row: int, first: int, pages) -> None:
        """Table entries ``first``.. of a row take new values; the change is noted for the device's copy."""
        g = self.groups[gi]
        g.tables[row, first:first + len(pages)] = pages
        base = row * self.max_pages_per_request + first
        changed = self._changed[gi]
        for k, p in enumerate(pages):
            changed[base + k] = int(p)

    def pages_to_grow(self, req_id, new_len: int) -> List[int]:
        """Pages each group must hand out so that the request can hold ``new_len`` tokens."""
        h = self._held[req_id]
        need = -(-new_len // self.page_size)
        return [max(0, need - h.next_page[i]) for i in range(len(self.groups))]

    def can_grow(self, req_id, new_len: int, reserve: int = 0) -> bool:
        """True if every group has the pages for ``new_len`` tokens and ``reserve`` more."""
        if new_len > self.max_len:
            return False
        return all(g.allocator.num_free() >= n + reserve for g, n in zip(self.groups, self.pages_to_grow(req_id, new_len)))

    def tokens_that_fit(self, req_id, reserve: int = 0) -> int:
        """How many more tokens than it has stored the request could hold with the free pages of every group,
        ``reserve`` of them left alone."""
        h = self._held[req_id]
        fit = self.max_len - h.computed
        for i, g in enumerate(self.groups):
            room = (h.next_page[i] + max(0, g.allocator.num_free() - reserve)) * self.page_size - h.computed
            fit = min(fit, room)
        return fit

    def grow(self, req_id, new_len: int) -> None:
        """Allocate pages in every group for tokens up to ``new_len``; all groups or none."""
        if new_len > self.max_len:
            raise ValueError(f"request {req_id!r} would hold {new_len} tokens; the tables are made for {self.max_len}")
        h = self._held[req_id]
        needs = self.pages_to_grow(req_id, new_len)
        for g, n in zip(self.groups, needs):
            if g.allocator.num_free() < n:
                raise OutOfPages(f"request {req_id!r} needs {n} pages for {new_len} tokens, "
                                 f"{g.allocator.num_free()} are free")
        for i, (g, n) in enumerate(zip(self.groups, needs)):
            if n:
                self._set(i, h.row, h.next_page[i], [g.allocator.allocate() for _ in range(n)])
                h.next_page[i] += n

    def advance(self, req_id, computed: int) -> None:
        """``computed`` tokens are stored now; windowed groups give back the pages the window has passed."""
        h = self._held[req_id]
        if computed < h.computed:
            raise ValueError("a request's stored tokens cannot shrink; free it and add it again")
        if self.groups and computed > min(h.next_page) * self.page_size:
            raise ValueError(f"request {req_id!r}: {computed} tokens stored but pages for fewer were allocated")
        h.computed = computed
        for i, g in enumerate(self.groups):
            first = min(self._first_needed(g, computed), h.next_page[i])
            if first > h.first_live[i]:
                for p in range(h.first_live[i], first):
                    g.allocator.decref(int(g.tables[h.row, p]))
                self._set(i, h.row, h.first_live[i], [NULL_PAGE] * (first - h.first_live[i]))
                h.first_live[i] = first

    def free(self, req_id) -> None:
        """Give back everything the request holds."""
        h = self._held.pop(req_id)
        for i, g in enumerate(self.groups):
            for p in range(h.first_live[i], h.next_page[i]):
                g.allocator.decref(int(g.tables[h.row, p]))
            if h.next_page[i] > h.first_live[i]:
                self._set(i, h.row, h.first_live[i], [NULL_PAGE] * (h.next_page[i] - h.first_live[i]))
        self._free_rows.append(h.row)

    def pages_held(self, req_id) -> List[List[int]]:
        h = self._held[req_id]
        return [[int(x) for x in g.tables[h.row, h.first_live[i]:h.next_page[i]]] for i, g in enumerate(self.groups)]

    def num_free_pages(self) -> List[int]:
        return [g.allocator.num_free() for g in self.groups]

    # ------------------------------------------------------------------ the device's copy of the tables
    def pending_updates(self) -> int:
        """The most entries any group's table has changed by since ``take_updates``."""
        return max((len(c) for c in self._changed), default=0)

    def take_updates(self) -> List[Tuple[np.ndarray, np.ndarray]]:
        """Per group (flat indices into the [rows, pages] table, their new values), each index once, and forget
        them: applied to a copy of the tables in this order of calls, the copy equals ``groups[g].tables``."""
        out = []
        for c in self._changed:
            out.append((np.fromiter(c.keys(), dtype=np.int32, count=len(c)),
                        np.fromiter(c.values(), dtype=np.int32, count=len(c))))
            c.clear()
        return out

    # ------------------------------------------------------------------ accounting
    def bytes_per_token(self, bytes_per_value: int) -> int:
        return self.layout.bytes_per_token(bytes_per_value)

    def check_invariants(self) -> None:
        """No page lost, held twice or freed twice; rows are held once; tables agree with the allocators."""
        rows = [h.row for h in self._held.values()]
        assert len(rows) == len(set(rows)), "a row is held by two requests"
        assert sorted(rows + self._free_rows) == list(range(self.max_requests)), "a row was lost"
        for i, g in enumerate(self.groups):
            g.allocator.check_invariants()
            owners: Dict[int, int] = {}
            for h in self._held.values():
                live = g.tables[h.row, h.first_live[i]:h.next_page[i]]
                assert (live != NULL_PAGE).all(), "a live table entry is the null page"
                assert (g.tables[h.row, :h.first_live[i]] == NULL_PAGE).all(), "a passed page is still in the table"
                assert (g.tables[h.row, h.next_page[i]:] == NULL_PAGE).all(), "the table holds a page beyond its end"
                for p in live:
                    owners[int(p)] = owners.get(int(p), 0) + 1
            for r in self._free_rows + [self.null_row]:
                assert (g.tables[r] == NULL_PAGE).all(), "a free row still holds pages"
            for p in range(1, g.allocator.num_pages + 1):
                assert g.allocator.ref[p] == owners.get(p, 0), \
                    f"group {i} page {p}: count {g.allocator.ref[p]} but {owners.get(p, 0)} table entries"
