"""Builds the flat description of a step's batch that the kernels read.

A step is a list of (request, its next tokens, the places among them whose logits are wanted): portions
of prompts beside single decoded tokens, cut anywhere.  The reference has no such thing: its forward takes
a rectangle of B rows by T tokens (src/miniserve/model.py:208-237) and a per-call cache view that builds
positions, a padded block table and a boolean mask (src/miniserve/paged.py:184-201).  Here positions,
the token-to-request map, per-group block tables and slot mappings are computed once on the host, packed
into one int32 array and sent in one copy; the mask is implicit (key j is visible to a token at position p
iff j <= p, and within the window if there is one).
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass
from typing import Hashable, List, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..parts.base import StepContext


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices into ``tokens``


class BatchBuilder:
    def __init__(self, manager: CacheManager, vocab_size: int, device):
        self.manager, self.vocab_size, self.device = manager, vocab_size, device

    def build(self, entries: List[StepEntry]):
        """Returns (StepContext, per-group block tables, per-group slot mappings).  Pages for the new
        tokens must already be allocated (``CacheManager.grow``)."""
        m = self.manager
        ps = m.page_size
        R = len(entries)
        q_lens = [len(e.tokens) for e in entries]
        if R == 0 or min(q_lens) <= 0:
            raise ValueError("a step needs at least one entry and every entry at least one token")
        N = sum(q_lens)
        rows = np.fromiter((m.row(e.req_id) for e in entries), dtype=np.int32, count=R)
        starts = np.fromiter((m.computed(e.req_id) for e in entries), dtype=np.int32, count=R)
        lens = np.asarray(q_lens, dtype=np.int32)
        ctx_lens = starts + lens
        if int(ctx_lens.max()) > m.max_len:
            raise ValueError(f"a request would hold {int(ctx_lens.max())} tokens; the cache is made for {m.max_len}")
        q_start = np.zeros(R + 1, dtype=np.int32)
        np.cumsum(lens, out=q_start[1:])
        token_ids = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=N)
        if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
            bad = int(token_ids[(token_ids < 0) | (token_ids >= self.vocab_size)][0])
            raise ValueError(f"token id {bad} is outside the vocabulary of {self.vocab_size}")
        token_req = np.repeat(np.arange(R, dtype=np.int32), lens)
        positions = np.arange(N, dtype=np.int32) - np.repeat(q_start[:-1], lens) + np.repeat(starts, lens)
        logit_rows = []
        for r, e in enumerate(entries):
            for w in e.want:
                if not 0 <= w < q_lens[r]:
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is not among its {q_lens[r]} tokens")
                logit_rows.append(int(q_start[r]) + int(w))
        logit_rows = np.asarray(logit_rows, dtype=np.int32)
        max_ctx = int(ctx_lens.max())
        n_pages = -(-max_ctx // ps)
        tables, slots = [], []
        for g in m.groups:
            t = g.tables[rows, :n_pages]
            page = t[token_req, positions // ps]
            if (page == 0).any():
                raise RuntimeError("a token of this step has no page; grow the request before building the batch")
            tables.append(np.ascontiguousarray(t))
            slots.append(page.astype(np.int32) * ps + positions % ps)

        parts = [token_ids.astype(np.int32), positions, token_req, q_start, ctx_lens, rows, logit_rows]
        parts += [t.reshape(-1) for t in tables] + slots
        sizes = [p.size for p in parts]
        packed = np.concatenate(parts) if N else np.zeros(0, np.int32)
        dev = torch.from_numpy(packed).to(self.device)
        views, off = [], 0
        for s in sizes:
            views.append(dev[off:off + s])
            off += s
        ng = len(m.groups)
        ctx = StepContext(
            num_tokens=N, num_requests=R, token_ids=views[0], positions=views[1], token_req=views[2],
            q_start=views[3], context_lens=views[4], state_slots=views[5], logit_rows=views[6],
            max_q_len=int(lens.max()), max_context_len=max_ctx, q_lens_host=q_lens,
            start_pos_host=[int(s) for s in starts], state_slots_host=[int(r) for r in rows])
        dev_tables = [views[7 + i].view(R, n_pages) for i in range(ng)]
        dev_slots = views[7 + ng:7 + 2 * ng]
        return ctx, dev_tables, dev_slots
