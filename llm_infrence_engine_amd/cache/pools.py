"""Device memory of the cache: per group and page tensor one tensor for every run that keeps its cache
there, and per stateful run its tensors of per-request slots.

A page tensor is [num_pages + 1, heads, page_size, width] (for keys and values the layout of
src/miniserve/paged.py:139-155, which keeps a head's page_size keys contiguous); page 0 is the null page.
A page tensor whose mixer asked for it (``PageTensor.transpose_at``, the matrix-core attention does for its
values in bfloat16) is kept transposed, [num_pages + 1, heads, width, page_size], when the page size allows.
State tensors have one slot more than there are request rows: the last belongs to nobody, and rows that pad
a captured batch point there.  The block tables are here too, one int32 [request rows + 1, pages per request]
per group, kept in step with the cache manager's by the entries that changed (``apply_updates``); the
reference builds and uploads a padded table on every forward (src/miniserve/paged.py:188-194).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import torch

from ..kernels import ops
from ..parts.base import KVView, Runtime, StateView
from .manager import CacheLayout


class CachePools:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages, max_requests: int, rt: Runtime,
                 max_pages_per_request: int = 1):
        """``num_pages``: usable pages of every group's pool, or one number per group."""
        n_groups = len(layout.group_keys)
        per_group = [int(num_pages)] * n_groups if isinstance(num_pages, int) else [int(n) for n in num_pages]
        if len(per_group) != n_groups:
            raise ValueError(f"{len(per_group)} pool sizes for {n_groups} cache groups")
        self.layout, self.page_size, self.max_requests = layout, page_size, max_requests
        self.pages_per_group = per_group
        self.pages: List[Dict[str, torch.Tensor]] = []   # per group: name -> [entries, pages + 1, heads, ., .]
        self.transposed: List[Dict[str, bool]] = []
        self.tables: List[torch.Tensor] = [
            torch.zeros((max_requests + 1, max_pages_per_request), dtype=torch.int32, device=rt.device)
            for _ in range(n_groups)]
        for (key, runs), num_pages in zip(zip(layout.group_keys, layout.group_runs), per_group):
            tensors, flipped = {}, {}
            for t in key.tensors:
                flipped[t.name] = (t.transpose_at is not None and page_size % t.transpose_at == 0
                                   and t.transpose_in in (None, rt.dtype))
                inner = (t.width, page_size) if flipped[t.name] else (page_size, t.width)
                tensors[t.name] = torch.zeros((len(runs), num_pages + 1, t.heads, *inner), dtype=rt.dtype, device=rt.device)
            self.pages.append(tensors)
            self.transposed.append(flipped)
        self.null_state_slot = max_requests
        self.state: Dict[int, tuple] = {}
        for run, need in layout.state_needs.items():
            needs = need if isinstance(need, tuple) else (need,)
            self.state[run] = tuple(torch.zeros((max_requests + 1, *n.shape), dtype=n.dtype, device=rt.device) for n in needs)

    def total_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for g in self.pages for t in g.values()) + \
            sum(t.numel() * t.element_size() for ts in self.state.values() for t in ts)

    def kv_view(self, run: int, table_rows: torch.Tensor, slot_mapping: torch.Tensor) -> KVView:
        """The run's pages with its group's table; ``table_rows`` [R]: the rows of the step's requests."""
        g, e = self.layout.run_group[run], self.layout.run_entry[run]
        return KVView({name: t[e] for name, t in self.pages[g].items()}, dict(self.transposed[g]), self.tables[g],
                      slot_mapping, store=self.layout.run_stores[run], window=self.layout.group_keys[g].window,
                      table_rows=table_rows)

    def apply_updates(self, index: Sequence[torch.Tensor], value: Sequence[torch.Tensor], counts: torch.Tensor,
                      max_updates: int) -> None:
        """Table entries that changed, as the cache manager's ``take_updates`` lists them (device tensors)."""
        ops.table_update(self.tables, list(index), list(value), counts, max_updates)

    def state_view(self, run: int) -> StateView:
        need = self.layout.state_needs[run]
        return StateView(self.state[run] if isinstance(need, tuple) else self.state[run][0])

    def zero_state(self, rows: torch.Tensor, count: Optional[torch.Tensor] = None) -> None:
        """A request's first portion starts from zero state: the slots ``rows`` (device int32; with ``count``, a
        device int, the first that many of them) of every state tensor."""
        if rows.numel() == 0:
            return
        for ts in self.state.values():
            for t in ts:
                ops.zero_rows(t, rows, count)
