"""Device memory of the cache: per group and page tensor one tensor for every run that keeps its cache
there, and per stateful run its tensors of per-request slots.

A page tensor is [num_pages + 1, heads, page_size, width] (for keys and values the layout of
src/miniserve/paged.py:139-155, which keeps a head's page_size keys contiguous); page 0 is the null page.
A page tensor whose mixer asked for it (``PageTensor.transpose_at``, the matrix-core attention does for its
values in bfloat16) is kept transposed, [num_pages + 1, heads, width, page_size], when the page size allows.
State tensors have one slot more than there are request rows: the last belongs to nobody, and rows that pad
a captured batch point there.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..parts.base import KVView, Runtime, StateView
from .manager import CacheLayout


class CachePools:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages: int, max_requests: int, rt: Runtime):
        self.layout, self.page_size, self.num_pages, self.max_requests = layout, page_size, num_pages, max_requests
        self.pages: List[Dict[str, torch.Tensor]] = []   # per group: name -> [entries, pages + 1, heads, ., .]
        self.transposed: List[Dict[str, bool]] = []
        for key, runs in zip(layout.group_keys, layout.group_runs):
            tensors, flipped = {}, {}
            for t in key.tensors:
                flipped[t.name] = t.transpose_at is not None and page_size % t.transpose_at == 0
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

    def kv_view(self, run: int, block_table: torch.Tensor, slot_mapping: torch.Tensor) -> KVView:
        g, e = self.layout.run_group[run], self.layout.run_entry[run]
        return KVView({name: t[e] for name, t in self.pages[g].items()}, dict(self.transposed[g]), block_table,
                      slot_mapping, store=self.layout.run_stores[run], window=self.layout.group_keys[g].window)

    def state_view(self, run: int) -> StateView:
        need = self.layout.state_needs[run]
        return StateView(self.state[run] if isinstance(need, tuple) else self.state[run][0])

    def zero_state(self, rows: List[int]) -> None:
        """A request's first portion starts from zero state."""
        if rows and self.state:
            idx = torch.tensor(rows, dtype=torch.long, device=next(iter(self.state.values()))[0].device)
            for ts in self.state.values():
                for t in ts:
                    t.index_fill_(0, idx, 0)
