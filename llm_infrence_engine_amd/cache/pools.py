"""Device memory of the cache: per group one tensor of pages for every run that keeps its cache there,
and per stateful run one tensor of per-request slots.

Pages are [num_pages + 1, kv heads, page_size, head size] for keys and the same for values (the layout of
src/miniserve/paged.py:139-155, which keeps a head's page_size keys contiguous); page 0 is the null page.
In bfloat16 with pages of a multiple of 16 tokens the value pages are kept transposed,
[num_pages + 1, kv heads, head size, page_size]: the matrix-core attention reads them as an operand as they lie.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from ..parts.base import KVView, Runtime, StateView
from .manager import CacheLayout


class CachePools:
    def __init__(self, layout: CacheLayout, page_size: int, num_pages: int, max_requests: int, rt: Runtime):
        self.layout, self.page_size, self.num_pages = layout, page_size, num_pages
        self.v_transposed = rt.dtype == torch.bfloat16 and page_size % 16 == 0
        self.kv: List[torch.Tensor] = []   # per group [entries, 2, pages + 1, nkv, page_size, d]
        for key, runs in zip(layout.group_keys, layout.group_runs):
            self.kv.append(torch.zeros((len(runs), 2, num_pages + 1, key.num_kv_heads, page_size, key.head_dim),
                                       dtype=rt.dtype, device=rt.device))
        self.state: Dict[int, torch.Tensor] = {
            run: torch.zeros((max_requests, *need.shape), dtype=need.dtype, device=rt.device)
            for run, need in layout.state_needs.items()}

    def total_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.kv) + \
            sum(t.numel() * t.element_size() for t in self.state.values())

    def kv_view(self, run: int, block_table: torch.Tensor, slot_mapping: torch.Tensor) -> KVView:
        g, e = self.layout.run_group[run], self.layout.run_entry[run]
        pages = self.kv[g][e]
        v = pages[1]
        if self.v_transposed:
            P, nkv, ps, d = v.shape
            v = v.view(P, nkv, d, ps)
        return KVView(pages[0], v, block_table, slot_mapping, store=self.layout.run_stores[run],
                      window=self.layout.group_keys[g].window, v_transposed=self.v_transposed)

    def state_view(self, run: int) -> StateView:
        return StateView(self.state[run])

    def zero_state(self, rows: List[int]) -> None:
        """A request's first portion starts from zero state."""
        if rows and self.state:
            idx = torch.tensor(rows, dtype=torch.long, device=next(iter(self.state.values())).device)
            for t in self.state.values():
                t.index_fill_(0, idx, 0)
