"""The flat description of a step's batch that the kernels read, and the one place that builds it.

A step is a list of (request, its next tokens, the places among them whose logits are wanted): portions
of prompts beside single decoded tokens, cut anywhere.  The reference has no such thing: its forward takes
a rectangle of B rows by T tokens (src/miniserve/model.py:208-237) and a per-call cache view that builds
positions, a padded block table and a boolean mask on the CPU (src/miniserve/paged.py:184-201).  Here the
description is one int32 array (``StepLayout`` says where each field lies) that is filled in pinned host
memory and sent in one asynchronous copy.  The block tables are not part of it: they live on the device
(``CachePools.tables``) and a step brings only the entries that changed since the last one.  The mask is
implicit (key j is visible to a token at position p iff j <= p, and within the window if there is one).

The same builder serves a step that is launched kernel by kernel (fields exactly as long as the step needs)
and a step that is replayed from a captured graph (``engine/graph.py``: fields of a fixed capacity, padded):
a padding token belongs to no request and stores nothing, a padding request has no tokens, no keys and
nobody's state slot.
"""
from __future__ import annotations

import itertools
from dataclasses import dataclass
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..cache.pools import CachePools
from ..parts.base import StepContext


@dataclass
class StepEntry:
    req_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices into ``tokens``


class StepLayout:
    """Where the fields of a step's description lie in its int32 array, for ``n_tokens`` tokens of ``n_requests``
    requests with ``n_wanted`` logit rows, ``n_groups`` cache groups and room for ``n_updates`` changed table
    entries per group.  A new per-token or per-request field is added here, in ``BatchBuilder.write`` and (if
    it moves from one decode step to the next) in the ``decode_advance`` kernel; nowhere else."""

    def __init__(self, n_tokens: int, n_requests: int, n_wanted: int, n_groups: int, n_updates: int):
        self.n_tokens, self.n_requests, self.n_wanted = n_tokens, n_requests, n_wanted
        self.n_groups, self.n_updates = n_groups, n_updates
        self.at: Dict[str, slice] = {}
        o = 0
        fields = [("token_ids", n_tokens), ("positions", n_tokens), ("token_req", n_tokens)]
        fields += [(f"slots{g}", n_tokens) for g in range(n_groups)]
        fields += [("q_start", n_requests + 1), ("context_lens", n_requests), ("state_slots", n_requests),
                   ("fresh_rows", n_requests), ("logit_rows", n_wanted), ("n_live", 1), ("n_fresh", 1),
                   ("update_counts", n_groups)]
        for g in range(n_groups):
            fields += [(f"update_index{g}", n_updates), (f"update_value{g}", n_updates)]
        # how each request's next token is chosen, for steps that choose it on the device: float fields hold the
        # bits of a float32, "seeds" two ints to a request (one int64, at an even offset)
        fields += [("seeds", 2 * n_requests), ("temperature", n_requests), ("top_p", n_requests), ("top_k", n_requests),
                   ("draw_index", n_requests)]
        for name, n in fields:
            if name == "seeds":
                o += o & 1
            self.at[name] = slice(o, o + n)
            o += n
        self.size = o


class StepBuffers:
    """A pinned host array and its device twin; ``send`` copies the first ``n`` ints over without waiting."""

    def __init__(self, size: int, device):
        self.size = size
        self.host = torch.zeros(max(1, size), dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(max(1, size), dtype=torch.int32, device=device)
        self._sent: Optional[torch.cuda.Event] = None

    def wait_until_sent(self) -> None:
        """The last copy must have read the pinned array before it is written again."""
        if self._sent is not None:
            self._sent.synchronize()

    def send(self, n: Optional[int] = None) -> None:
        n = self.size if n is None else n
        if n:
            self.dev[:n].copy_(self.host[:n], non_blocking=True)
        if self._sent is None:
            self._sent = torch.cuda.Event()
        self._sent.record()

    def views(self, layout: StepLayout) -> Dict[str, torch.Tensor]:
        v = {name: self.dev[sl] for name, sl in layout.at.items()}
        v["temperature"], v["top_p"] = v["temperature"].view(torch.float32), v["top_p"].view(torch.float32)
        v["seeds"] = v["seeds"].view(torch.int64)
        return v


@dataclass
class _Described:
    """A step's live part as host arrays."""

    n_tokens: int
    n_requests: int
    token_ids: np.ndarray
    positions: np.ndarray
    token_req: np.ndarray
    slots: List[np.ndarray]
    q_start: np.ndarray
    context_lens: np.ndarray
    rows: np.ndarray
    fresh_rows: np.ndarray
    logit_rows: np.ndarray
    q_lens: List[int]
    starts: np.ndarray
    sampling: Optional[Sequence] = None    # per request (temperature, top_k, top_p, seed, draw index), or None: greedy


@dataclass
class Sampling:
    """How one request's next token is chosen on the device (``sampling/sampler.py`` has the rules)."""

    temperature: float = 0.0
    top_k: int = 0
    top_p: float = 1.0
    seed: int = 0
    draw_index: int = 0


@dataclass
class BuiltStep:
    ctx: StepContext
    slots: List[torch.Tensor]          # per cache group, int32 [N]
    fields: Dict[str, torch.Tensor]    # every field of the layout as a device view


class BatchBuilder:
    def __init__(self, manager: CacheManager, pools: CachePools, vocab_size: int, device):
        self.manager, self.pools, self.vocab_size, self.device = manager, pools, vocab_size, device
        # steps that are launched kernel by kernel alternate between two arrays, so that filling the next one
        # never waits for the copy of the last
        self._arena: List[Optional[StepBuffers]] = [None, None]
        self._turn = 0

    # ------------------------------------------------------------------ what a step holds
    def describe(self, entries: List[StepEntry], steps: int = 1) -> _Described:
        """Host arrays for ``entries``; pages for their tokens (and, with ``steps`` > 1, for the decode steps that
        follow on the device) must already be allocated (``CacheManager.grow``)."""
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
        longest = int(ctx_lens.max()) + steps - 1
        if longest > m.max_len:
            raise ValueError(f"a request would hold {longest} tokens; the cache is made for {m.max_len}")
        q_start = np.zeros(R + 1, dtype=np.int32)
        np.cumsum(lens, out=q_start[1:])
        token_ids = np.fromiter(itertools.chain.from_iterable(e.tokens for e in entries), dtype=np.int64, count=N)
        if token_ids.min() < 0 or token_ids.max() >= self.vocab_size:
            bad = int(token_ids[(token_ids < 0) | (token_ids >= self.vocab_size)][0])
            raise ValueError(f"token id {bad} is outside the vocabulary of {self.vocab_size}")
        token_req = np.repeat(np.arange(R, dtype=np.int32), lens)
        positions = np.arange(N, dtype=np.int32) - np.repeat(q_start[:-1], lens) + np.repeat(starts, lens)
        wanted = []
        for r, e in enumerate(entries):
            for w in e.want:
                if not 0 <= w < q_lens[r]:
                    raise ValueError(f"request {e.req_id!r}: wanted place {w} is not among its {q_lens[r]} tokens")
                wanted.append(int(q_start[r]) + int(w))
        slots = []
        token_rows = rows[token_req]
        last_page = (ctx_lens + steps - 2) // ps
        for g in m.groups:
            page = g.tables[token_rows, positions // ps]
            if (page == 0).any() or (g.tables[rows, last_page] == 0).any():
                raise RuntimeError("a token of this step has no page; grow the request before building the batch")
            slots.append(page.astype(np.int32) * ps + positions % ps)
        return _Described(N, R, token_ids.astype(np.int32), positions, token_req, slots, q_start, ctx_lens, rows,
                          rows[starts == 0], np.asarray(wanted, dtype=np.int32), q_lens, starts)

    # ------------------------------------------------------------------ into an array
    def write(self, d: Optional[_Described], layout: StepLayout, a: np.ndarray) -> int:
        """Fill ``a`` (the host array of a layout at least as large as the step) and return how many changed table
        entries it brings.  Fields longer than the step are padded: tokens that belong to no request and store
        nothing, requests without tokens or keys on nobody's row, wanted rows that repeat row 0."""
        m, at = self.manager, layout.at
        N = d.n_tokens if d else 0
        R = d.n_requests if d else 0
        if N > layout.n_tokens or R > layout.n_requests or (d is not None and d.logit_rows.size > layout.n_wanted):
            raise ValueError("the step does not fit the layout it is written into")

        def put(name, values, pad):
            f = a[at[name]]
            n = len(values)
            f[:n] = values
            if n < f.size:
                f[n:] = pad

        empty = np.zeros(0, np.int32)
        put("token_ids", d.token_ids if d else empty, 0)
        put("positions", d.positions if d else empty, 0)
        put("token_req", d.token_req if d else empty, 0)
        for g in range(layout.n_groups):
            put(f"slots{g}", d.slots[g] if d else empty, -1)
        put("q_start", d.q_start if d else np.zeros(1, np.int32), N)
        put("context_lens", d.context_lens if d else empty, 0)
        put("state_slots", d.rows if d else empty, m.null_row)
        put("fresh_rows", d.fresh_rows if d else empty, m.null_row)
        put("logit_rows", d.logit_rows if d else empty, 0)
        a[at["n_live"]] = R
        a[at["n_fresh"]] = d.fresh_rows.size if d else 0
        how = list(d.sampling) if d is not None and d.sampling is not None else []
        if how and len(how) != R:
            raise ValueError("one Sampling per request of the step, or none")
        put("temperature", np.asarray([h.temperature for h in how], dtype=np.float32).view(np.int32), 0)
        put("top_p", np.asarray([h.top_p for h in how], dtype=np.float32).view(np.int32), 0)
        put("top_k", np.asarray([h.top_k for h in how], dtype=np.int32), 0)
        put("draw_index", np.asarray([h.draw_index for h in how], dtype=np.int32), 0)
        put("seeds", np.asarray([h.seed & 0x7FFFFFFFFFFFFFFF for h in how], dtype=np.int64).view(np.int32), 0)
        most = 0
        if m.pending_updates() > layout.n_updates:
            raise RuntimeError("more table entries changed than the layout has room for; flush them first")
        for g, (index, value) in enumerate(m.take_updates()):
            put(f"update_index{g}", index, -1)
            put(f"update_value{g}", value, 0)
            a[at["update_counts"]][g] = index.size
            most = max(most, index.size)
        return most

    def context(self, fields: Dict[str, torch.Tensor], n_tokens: int, n_requests: int, max_q_len: int,
                max_context_len: int, d: Optional[_Described] = None, padded: bool = False) -> StepContext:
        """The ``StepContext`` over the device views ``fields``.  ``d``: the step's host arrays, for the host copies
        that parts written in plain tensor code read (a captured step has none)."""
        R = n_requests
        return StepContext(
            num_tokens=n_tokens, num_requests=R, token_ids=fields["token_ids"], positions=fields["positions"],
            token_req=fields["token_req"], q_start=fields["q_start"], context_lens=fields["context_lens"],
            state_slots=fields["state_slots"], logit_rows=fields["logit_rows"], max_q_len=max_q_len,
            max_context_len=max_context_len,
            n_live_tokens=fields["q_start"][R:R + 1] if padded else None,
            q_lens_host=list(d.q_lens) if d else [], start_pos_host=[int(s) for s in d.starts] if d else [],
            state_slots_host=[int(r) for r in d.rows] if d else [])

    # ------------------------------------------------------------------ a step launched kernel by kernel
    def _next_buffers(self, size: int) -> StepBuffers:
        self._turn ^= 1
        buf = self._arena[self._turn]
        if buf is None or buf.size < size:
            buf = self._arena[self._turn] = StepBuffers(max(4096, 2 * size), self.device)
        buf.wait_until_sent()
        return buf

    def build(self, entries: List[StepEntry]) -> BuiltStep:
        """Describe ``entries`` exactly (no padding), send the description, bring the device's block tables up to
        date and zero the state slots of requests that start."""
        d = self.describe(entries)
        layout = StepLayout(d.n_tokens, d.n_requests, d.logit_rows.size, len(self.manager.groups),
                            self.manager.pending_updates())
        buf = self._next_buffers(layout.size)
        n_updates = self.write(d, layout, buf.np)
        buf.send(layout.size)
        fields = buf.views(layout)
        self._apply(fields, layout, n_updates, d.fresh_rows.size)
        ctx = self.context(fields, d.n_tokens, d.n_requests, max(d.q_lens), int(d.context_lens.max()), d)
        return BuiltStep(ctx, [fields[f"slots{g}"] for g in range(layout.n_groups)], fields)

    def _apply(self, fields, layout: StepLayout, n_updates: int, n_fresh: int) -> None:
        G = layout.n_groups
        if n_updates:
            self.pools.apply_updates([fields[f"update_index{g}"] for g in range(G)],
                                     [fields[f"update_value{g}"] for g in range(G)], fields["update_counts"],
                                     layout.n_updates)
        if n_fresh and self.pools.state:
            self.pools.zero_state(fields["fresh_rows"][:n_fresh])

    def flush_updates(self) -> None:
        """Bring the device's block tables up to date now, outside any step (before a captured step whose
        description has no room for all the entries that changed)."""
        if not self.manager.pending_updates():
            return
        layout = StepLayout(0, 0, 0, len(self.manager.groups), self.manager.pending_updates())
        buf = self._next_buffers(layout.size)
        n_updates = self.write(None, layout, buf.np)
        buf.send(layout.size)
        self._apply(buf.views(layout), layout, n_updates, 0)
