"""Decode-only steps replayed from captured HIP graphs, one graph per batch-size bucket.

A decode step of a small model is bound by kernel launches, not by the GPU (the reference measured the
same on its hardware and answered with CUDA graphs, src/miniserve/graph_decode.py:33-86).  The whole
forward of a batch of single tokens is captured once per bucket {1, 2, 4, ..., max} (graph_decode.py:23-30)
over static input buffers; a step then fills a pinned host copy of those buffers, sends it in one copy and
replays.  Nothing in the captured kernels depends on how long the contexts are (block tables have their
full width, the attention kernel spreads each request's keys over its waves itself), so a graph stays valid
for the life of the engine; only the choice between the attention's two launch shapes (contexts up to
``ops.LONG_CONTEXT`` or beyond) is made per step, and each has graphs of its own.  Rows that pad a batch up to its bucket read the null page and store nothing.
The greedy choice (argmax) of every row is part of the graph.

A graph may also hold several decode steps in a row: between two steps a small kernel moves every live
request one position on, feeds it the token just chosen and looks up its new slots in the block tables, all
on the device, so the host is needed once per launch instead of once per step.
"""
from __future__ import annotations

import gc
import time
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from ..parts.base import StepContext
from ..parts.model import RunCache
from .batch import StepEntry


def default_batch_sizes(max_batch: int) -> List[int]:
    """The batch-size buckets graphs are captured for: every power of two below ``max_batch`` and ``max_batch``
    itself, the rule the reference states for its own buckets (src/miniserve/graph_decode.py:23-30;
    8 -> 1, 2, 4, 8 and 6 -> 1, 2, 4, 6 in its tests/test_cuda_graph.py:45-48)."""
    if max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    return sorted({1 << e for e in range(max_batch.bit_length()) if (1 << e) < max_batch} | {max_batch})


class _Bucket:
    def __init__(self, B: int, width: int, n_groups: int, device, steps: int = 1, null_state_slot: int = 0):
        self.B, self.width, self.steps, self.null_state_slot = B, width, steps, null_state_slot
        # layout of the static int32 buffer
        self.off: Dict[str, slice] = {}
        o = 0
        for name, n in (("token_ids", B), ("positions", B), ("token_req", B), ("q_start", B + 1),
                        ("context_lens", B), ("state_slots", B), ("logit_rows", B), ("n_live", 1)):
            self.off[name] = slice(o, o + n)
            o += n
        self.tables, self.slots = [], []
        for g in range(n_groups):
            self.tables.append(slice(o, o + B * width)); o += B * width
            self.slots.append(slice(o, o + B)); o += B
        self.size = o
        self.host = torch.zeros(o, dtype=torch.int32).pin_memory()
        self.np = self.host.numpy()
        self.dev = torch.zeros(o, dtype=torch.int32, device=device)
        self.reset_host()
        self.dev.copy_(self.host)
        self.last_rows = 0
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.tokens = torch.zeros((steps, B), dtype=torch.int32, device=device)   # the argmax of every step
        self.copied: Optional[torch.cuda.Event] = None   # set once the last copy of ``host`` has left it

    def reset_host(self) -> None:
        """Every row a padding row: token 0 at position 0, one visible key on the null page, nothing stored."""
        a, B = self.np, self.B
        a[:] = 0
        a[self.off["token_req"]] = np.arange(B)
        a[self.off["q_start"]] = np.arange(B + 1)
        a[self.off["context_lens"]] = 1
        a[self.off["logit_rows"]] = np.arange(B)
        a[self.off["n_live"]] = 0
        a[self.off["state_slots"]] = self.null_state_slot      # nobody's slot
        for s in self.slots:
            a[s] = -1

    def context(self) -> StepContext:
        d, o = self.dev, self.off
        return StepContext(
            num_tokens=self.B, num_requests=self.B, token_ids=d[o["token_ids"]], positions=d[o["positions"]],
            token_req=d[o["token_req"]], q_start=d[o["q_start"]], context_lens=d[o["context_lens"]],
            state_slots=d[o["state_slots"]], logit_rows=d[o["logit_rows"]], max_q_len=1,
            max_context_len=self.width, q_lens_host=[1] * self.B, start_pos_host=[0] * self.B,
            state_slots_host=[self.null_state_slot] * self.B)


class DecodeGraphs:
    def __init__(self, runner, batch_sizes: Optional[Sequence[int]] = None):
        m = runner.manager
        if not runner.model.graph_safe():
            raise ValueError("HIP graphs are not used for this model: one of its parts says it cannot be captured "
                             "(Part.graph_safe)")
        self.runner, self.manager = runner, m
        self.sizes = sorted(set(batch_sizes or default_batch_sizes(m.max_requests)))
        self.width = m.max_pages_per_request
        self.buckets: Dict[tuple, _Bucket] = {}
        self.pool = None   # one memory pool for all graphs: they never run at the same time
        # what launching costs the host: seconds spent filling the buffers and enqueuing, and launches so far
        # (the reference separates a launch-bound from a GPU-bound step the same way, benchmarks/diag_gpu_launch.py:1-8)
        self.enqueue_seconds = 0.0
        self.launches = 0

    @property
    def max_batch(self) -> int:
        return self.sizes[-1]

    def context_classes(self) -> List[bool]:
        """The attention's launch shapes a decode step of this cache can need: short contexts, and long ones
        if a request can grow beyond ``ops.LONG_CONTEXT``."""
        return [False, True] if self.manager.max_len > ops.LONG_CONTEXT else [False]

    def warm_up(self, steps: Sequence[int] = (1,), batch_sizes: Optional[Sequence[int]] = None) -> int:
        """Capture, before serving, every graph that serving can reach: each batch-size bucket (or those of
        ``batch_sizes``), each context class, each number of steps per launch in ``steps``; the reference
        captures all its buckets in the constructor (src/miniserve/graph_decode.py:46-47).  Afterwards
        ``run`` captures nothing.  Returns the number of graphs held."""
        sizes = self.sizes if batch_sizes is None else sorted({next(b for b in self.sizes if b >= n) for n in batch_sizes})
        for B in reversed(sizes):            # the largest first: the others fit into the memory it leaves
            for long_context in self.context_classes():
                for k in sorted(set(steps), reverse=True):
                    self._bucket(B, long_context, k)
        return len(self.buckets)

    def _bucket(self, n: int, long_context: bool, steps: int = 1) -> _Bucket:
        B = next(b for b in self.sizes if b >= n)
        key = (B, long_context, steps)
        bk = self.buckets.get(key)
        if bk is None:
            bk = self.buckets[key] = _Bucket(B, self.width, len(self.manager.groups), self.runner.rt.device, steps,
                                             self.runner.pools.null_state_slot)
            self._capture(bk, long_context)
        return bk

    def _caches(self, bk: _Bucket) -> List[RunCache]:
        r = self.runner
        caches = []
        for i in range(len(r.model.spec.order)):
            g = r.layout.run_group[i]
            kv = None
            if g is not None:
                kv = r.pools.kv_view(i, bk.dev[bk.tables[g]].view(bk.B, bk.width), bk.dev[bk.slots[g]])
            state = r.pools.state_view(i) if i in r.layout.state_needs else None
            caches.append(RunCache(kv, state))
        return caches

    def _capture(self, bk: _Bucket, long_context: bool) -> None:
        ctx, caches = bk.context(), self._caches(bk)
        cap = self.width * self.manager.page_size
        ctx.max_context_len = cap if long_context else min(cap, ops.LONG_CONTEXT)
        model = self.runner.model
        d, o = bk.dev, bk.off
        tables = [d[s].view(bk.B, bk.width) for s in bk.tables]
        slots = [d[s] for s in bk.slots]

        def advance(k):   # n_live is 0 in the buffer while capturing and warming up: nothing moves
            ops.decode_advance(bk.tokens[k - 1], d[o["token_ids"]], d[o["positions"]], d[o["context_lens"]],
                               d[o["n_live"]], tables, slots, self.manager.page_size)

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            # load the kernels of this shape before capturing (twice for the first graph, which also
            # settles the allocator)
            for _ in range(1 if self.buckets.keys() - {(bk.B, long_context, bk.steps)} else 2):
                ops.sample(model.forward(ctx, caches), bk.tokens[0])
            if bk.steps > 1:
                advance(1)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        # Nothing that owns device memory or graphs of its own (a runner that went out of use and waits in a
        # reference cycle) may be finalised while the stream is capturing: giving device memory back is not
        # allowed then, and the error, raised inside a destructor, ends the process.  So the collector runs
        # now and stays off until the capture has ended.
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            if self.pool is None:
                self.pool = torch.cuda.graph_pool_handle()
            bk.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(bk.graph, pool=self.pool):
                for k in range(bk.steps):
                    if k > 0:
                        advance(k)
                    bk.logits = model.forward(ctx, caches)
                    ops.sample(bk.logits, bk.tokens[k])
        finally:
            if collecting:
                gc.enable()
        torch.cuda.synchronize()

    def run(self, entries: List[StepEntry], steps: int = 1):
        """``steps`` decode steps for ``entries`` (one token each, pages already grown for all the steps).
        Returns (logits [R, V] of the last step, greedy tokens int32 [steps, R]); both are views of static
        buffers that the next replay overwrites."""
        t_begin = time.perf_counter()
        m = self.manager
        R = len(entries)
        rows = np.fromiter((m.row(e.req_id) for e in entries), dtype=np.int32, count=R)
        pos = np.fromiter((m.computed(e.req_id) for e in entries), dtype=np.int32, count=R)
        bk = self._bucket(R, int(pos.max()) + steps > ops.LONG_CONTEXT, steps)
        a, o, ps = bk.np, bk.off, m.page_size
        if bk.copied is not None:
            bk.copied.synchronize()      # the last launch's copy must have read the pinned buffer before it changes
        toks = np.fromiter((e.tokens[0] for e in entries), dtype=np.int64, count=R)
        if toks.min() < 0 or toks.max() >= self.runner.model.spec.vocab_size:
            raise ValueError("a token id is outside the vocabulary")
        if int(pos.max()) + steps > m.max_len:
            raise ValueError(f"a request would hold {int(pos.max()) + steps} tokens; the cache is made for {m.max_len}")
        if R < bk.last_rows:
            bk.reset_host()
        bk.last_rows = R
        if self.runner.layout.state_runs and (pos == 0).any():
            self.runner.pools.zero_state([int(r) for r in rows[pos == 0]])      # a first token starts from zero state
        a[o["token_ids"]][:R] = toks
        a[o["positions"]][:R] = pos
        a[o["context_lens"]][:R] = pos + 1
        a[o["state_slots"]][:R] = rows
        a[o["n_live"]] = R
        used = (int(pos.max()) + steps - 1) // ps + 1
        for g, grp in enumerate(m.groups):
            t = a[bk.tables[g]].reshape(bk.B, bk.width)
            t[:R, :used] = grp.tables[rows, :used]
            page = t[np.arange(R), pos // ps]
            if (page == 0).any() or (t[np.arange(R), (pos + steps - 1) // ps] == 0).any():
                raise RuntimeError("a token of this launch has no page; grow the requests before it")
            a[bk.slots[g]][:R] = page * ps + pos % ps
        bk.dev.copy_(bk.host, non_blocking=True)
        if bk.copied is None:
            bk.copied = torch.cuda.Event()
        bk.copied.record()
        bk.graph.replay()
        self.enqueue_seconds += time.perf_counter() - t_begin
        self.launches += 1
        return bk.logits[:R], bk.tokens[:, :R]
