"""Steps replayed from captured HIP graphs.

A step of a small model is bound by kernel launches, not by the GPU (the reference measured the same on its
hardware and answered with CUDA graphs for its decode steps, src/miniserve/graph_decode.py:33-86).  Two kinds
of step are captured here, both over a static description of the batch (``engine/batch.py``: one int32 array
of fixed capacity per graph, padded by the same builder that describes a step launched kernel by kernel):

* decode steps, one graph per batch-size bucket {1, 2, 4, ..., max} (graph_decode.py:23-30): the whole
  forward of a batch of single tokens with the greedy choice (argmax) of every row.  A graph may hold several
  decode steps in a row: between two of them a small kernel moves every live request one position on, feeds
  it the token just chosen and looks up its new slots in the block tables, all on the device, so the host is
  needed once per launch instead of once per step;
* steps with prompt portions (alone or beside decoded tokens), one graph per bucket of the step's number of
  tokens: embedding and all layers; the final norm and the head run on the wanted rows afterwards, outside the
  graph, so that any number of rows may be wanted.  A short portion of a narrow model is over on the GPU
  before the host has enqueued its launches one by one; replayed, it costs the host one launch.

Nothing in the captured kernels depends on how the tokens are dealt out over the requests or on how long the
contexts are: the attention's launch is sized by the numbers of tokens and requests alone, block tables live on
the device with their full width, and the changed table entries and the state slots to zero travel in the
description.  So a graph stays valid for the life of the engine; only the choice between the decode
attention's two launch shapes (contexts up to ``ops.LONG_CONTEXT`` or beyond) is made per step, and each has
graphs of its own.
"""
from __future__ import annotations

import gc
import time
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from .batch import BatchBuilder, StepBuffers, StepEntry, StepLayout

PORTION_BUCKETS = (16, 32, 64, 128, 256, 384, 512, 768, 1024, 1536, 2048, 3072, 4096)


def default_batch_sizes(max_batch: int) -> List[int]:
    """The batch-size buckets graphs are captured for: every power of two below ``max_batch`` and ``max_batch``
    itself, the rule the reference states for its own buckets (src/miniserve/graph_decode.py:23-30;
    8 -> 1, 2, 4, 8 and 6 -> 1, 2, 4, 6 in its tests/test_cuda_graph.py:45-48)."""
    if max_batch < 1:
        raise ValueError("max_batch must be at least 1")
    return sorted({1 << e for e in range(max_batch.bit_length()) if (1 << e) < max_batch} | {max_batch})


def portion_graph_limit(model) -> int:
    """Up to how many tokens a step with prompt portions is worth replaying from a graph: as long as the GPU
    would be done before the host has enqueued the step's launches one by one (a few hundred launches at 10 to
    15 us each), at a rate of matrix work that short portions reach.  Beyond that the host hides behind the
    GPU anyway and a graph's padding up to its bucket would only add work."""
    weights = sum(s.shape[0] * s.shape[1] for s in model.tensor_specs() if s.role == "matrix" and len(s.shape) == 2)
    ends = sum(s.shape[0] * s.shape[1] for part in (model.embedding, model.head) for s in part.tensor_specs())
    per_token = 2.0 * max(1, weights - ends)
    launches = 9 * len(model.spec.order)
    tokens = launches * 13e-6 * 0.4e15 / per_token
    fits = [b for b in PORTION_BUCKETS if b <= tokens]
    return fits[-1] if fits else 0


class _Bucket:
    """One captured graph with the static description it reads."""

    def __init__(self, layout: StepLayout, device, steps: int = 1):
        self.layout, self.steps = layout, steps
        self.buf = StepBuffers(layout.size, device)
        self.fields = self.buf.views(layout)
        self.slots = [self.fields[f"slots{g}"] for g in range(layout.n_groups)]
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None       # decode: [rows, V] of the last step
        self.hidden = None                                # portions: (residual stream, unsummed addend)
        self.sampled = False                              # decode: False, or (top-k, top-p): tokens are drawn, not the argmax
        self.tokens = torch.zeros((steps, layout.n_requests), dtype=torch.int32, device=device)   # the argmax of every step


class StepGraphs:
    def __init__(self, runner, batch_sizes: Optional[Sequence[int]] = None, portion_tokens: Optional[int] = None):
        """``portion_tokens``: steps with prompt portions of up to that many tokens are replayed from graphs too
        (None: ``portion_graph_limit`` decides; 0: decode steps only)."""
        m = runner.manager
        if not runner.model.graph_safe():
            raise ValueError("HIP graphs are not used for this model: one of its parts says it cannot be captured "
                             "(Part.graph_safe)")
        self.runner, self.manager, self.builder = runner, m, runner.builder
        self.sizes = sorted(set(batch_sizes or default_batch_sizes(m.max_requests)))
        limit = portion_graph_limit(runner.model) if portion_tokens is None else portion_tokens
        if runner.model.graph_safe() is not True:      # a part that can be captured only while it decodes
            limit = 0
        self.portion_sizes = [b for b in PORTION_BUCKETS if b <= limit]
        self.width = m.max_pages_per_request
        self.buckets: Dict[tuple, _Bucket] = {}            # decode: (rows, long contexts, steps)
        self.portion_buckets: Dict[int, _Bucket] = {}      # steps with portions: tokens
        self.pool = None   # one memory pool for all graphs: they never run at the same time
        # what launching costs the host: seconds spent filling the buffers and enqueuing, and launches so far
        # (the reference separates a launch-bound from a GPU-bound step the same way, benchmarks/diag_gpu_launch.py:1-8)
        self.enqueue_seconds = 0.0
        self.launches = 0

    @property
    def max_batch(self) -> int:
        return self.sizes[-1]

    @property
    def max_portion_tokens(self) -> int:
        return self.portion_sizes[-1] if self.portion_sizes else 0

    def context_classes(self) -> List[bool]:
        """The attention's launch shapes a decode step of this cache can need: short contexts, and long ones
        if a request can grow beyond ``ops.LONG_CONTEXT``."""
        return [False, True] if self.manager.max_len > ops.LONG_CONTEXT else [False]

    def warm_up(self, steps: Sequence[int] = (1,), batch_sizes: Optional[Sequence[int]] = None,
                portion_tokens: Optional[Sequence[int]] = None) -> int:
        """Capture, before serving, every graph that serving can reach: each batch-size bucket (or those of
        ``batch_sizes``), each context class, each number of steps per launch in ``steps``, and each bucket of
        portion tokens (or those that ``portion_tokens`` fall into); the reference captures all its buckets in
        the constructor (src/miniserve/graph_decode.py:46-47).  Afterwards ``run`` captures nothing.  Returns
        the number of graphs held."""
        sizes = self.sizes if batch_sizes is None else sorted({next(b for b in self.sizes if b >= n) for n in batch_sizes})
        portions = self.portion_sizes if portion_tokens is None else \
            sorted({self._portion_size(n) for n in portion_tokens if self._portion_size(n)})
        for n in reversed(portions):         # the largest first: the others fit into the memory it leaves
            self._portion_bucket(n)
        for B in reversed(sizes):
            for long_context in self.context_classes():
                for k in sorted(set(steps), reverse=True):
                    self._bucket(B, long_context, k)
        return len(self.buckets) + len(self.portion_buckets)

    # ------------------------------------------------------------------ buckets
    def _bucket(self, n: int, long_context: bool, steps: int = 1, sampled=False) -> _Bucket:
        """``sampled``: False (the graph takes the argmax), or which thresholds the sampling kernels look for,
        (top-k, top-p): a graph of its own for each, so that rows which only have a temperature do not pay for
        the search."""
        B = next(b for b in self.sizes if b >= n)
        key = (B, long_context, steps) + (("sampled",) + tuple(sampled) if sampled else ())
        bk = self.buckets.get(key)
        if bk is None:
            ps = self.manager.page_size
            layout = StepLayout(B, B, B, len(self.manager.groups), B * (steps // ps + 2))
            bk = self.buckets[key] = _Bucket(layout, self.runner.rt.device, steps)
            bk.sampled = sampled
            cap = self.width * ps
            self._capture(bk, max_q_len=1, max_context_len=cap if long_context else min(cap, ops.LONG_CONTEXT))
        return bk

    def _portion_size(self, n_tokens: int) -> int:
        return next((b for b in self.portion_sizes if b >= n_tokens), 0)

    def _portion_bucket(self, size: int) -> _Bucket:
        bk = self.portion_buckets.get(size)
        if bk is None:
            m = self.manager
            R = m.max_requests
            layout = StepLayout(size, R, size, len(m.groups), size // m.page_size + 2 * R + 8)
            bk = self.portion_buckets[size] = _Bucket(layout, self.runner.rt.device)
            cap = self.width * m.page_size
            self._capture(bk, max_q_len=min(size, cap), max_context_len=cap)
        return bk

    def _capture(self, bk: _Bucket, max_q_len: int, max_context_len: int) -> None:
        lay, f = bk.layout, bk.fields
        runner, model = self.runner, self.runner.model
        decode = max_q_len == 1 and lay.n_tokens == lay.n_requests
        ctx = self.builder.context(f, lay.n_tokens, lay.n_requests, max_q_len, max_context_len, padded=True)
        caches = runner.caches(ctx.state_slots, bk.slots)
        G = lay.n_groups
        # what the table entries of the last steps changed must be on the device before a description that is all
        # padding stands in for a step
        self.builder.flush_updates()
        bk.buf.wait_until_sent()
        self.builder.write(None, lay, bk.buf.np)
        bk.buf.send()

        def body():
            ctx.shared.clear()     # what parts derive from the step's tensors is worked out inside every run
            if G:
                runner.pools.apply_updates([f[f"update_index{g}"] for g in range(G)],
                                           [f[f"update_value{g}"] for g in range(G)], f["update_counts"], lay.n_updates)
            if runner.pools.state:
                runner.pools.zero_state(f["fresh_rows"], f["n_fresh"])
            if not decode:
                bk.hidden = model.forward_hidden(ctx, caches)
                return
            for k in range(bk.steps):
                if k > 0:      # n_live is 0 in the buffer while capturing and warming up: nothing moves
                    ops.decode_advance(bk.tokens[k - 1], f["token_ids"], f["positions"], f["context_lens"], f["n_live"],
                                       f["state_slots"], runner.pools.tables, bk.slots, self.manager.page_size,
                                       f["draw_index"] if bk.sampled else None)
                    ctx.shared.clear()
                bk.logits = model.head_logits(*model.forward_hidden(ctx, caches), ctx.logit_rows)
                if bk.sampled:     # rows without a temperature (padding rows too) take the first maximum
                    ops.sample(bk.logits, bk.tokens[k], f["temperature"], f["top_k"], f["top_p"], f["seeds"], f["draw_index"],
                               use_top_k=bk.sampled[0], use_top_p=bk.sampled[1])
                else:
                    ops.sample(bk.logits, bk.tokens[k])

        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            # load the kernels of this shape before capturing (twice for the first graph, which also
            # settles the allocator)
            for _ in range(1 if self.pool is not None else 2):
                body()
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
                body()
        finally:
            if collecting:
                gc.enable()
        torch.cuda.synchronize()

    # ------------------------------------------------------------------ steps
    def takes(self, entries: List[StepEntry]) -> Optional[str]:
        """"decode", "portions", or None if the step is launched kernel by kernel."""
        if len(entries) <= self.max_batch and all(len(e.tokens) == 1 for e in entries):
            return "decode"
        if len(entries) <= self.manager.max_requests and self._portion_size(sum(len(e.tokens) for e in entries)):
            return "portions"
        return None

    def _fill_and_replay(self, bk: _Bucket, entries: List[StepEntry], steps: int, every_row: bool = False,
                         sampling=None):
        if self.manager.pending_updates() > bk.layout.n_updates:
            self.builder.flush_updates()
        d = self.builder.describe(entries, steps)
        d.sampling = sampling
        if every_row:     # a decode graph works out the logits and the greedy choice of every request, wanted or not
            d.logit_rows = np.arange(d.n_requests, dtype=np.int32)
        bk.buf.wait_until_sent()
        self.builder.write(d, bk.layout, bk.buf.np)
        bk.buf.send()
        bk.graph.replay()
        return d

    def run(self, entries: List[StepEntry], steps: int = 1, sampling=None):
        """``steps`` decode steps for ``entries`` (one token each, pages already grown for all the steps).
        ``sampling``: one ``batch.Sampling`` per entry if any of them draws its tokens (the graph then holds the
        sampling kernels instead of the argmax), else None.  Returns (logits [R, V] of the last step, chosen
        tokens int32 [steps, R]); both are views of static buffers that the next replay overwrites."""
        t_begin = time.perf_counter()
        R = len(entries)
        longest = max(self.manager.computed(e.req_id) for e in entries) + steps
        sampled = False
        if sampling is not None:
            V = self.runner.model.spec.vocab_size
            sampled = (any(0 < h.top_k < V for h in sampling), any(h.top_p < 1.0 for h in sampling))
        bk = self._bucket(R, longest > ops.LONG_CONTEXT, steps, sampled=sampled)
        self._fill_and_replay(bk, entries, steps, every_row=True, sampling=sampling)
        self.enqueue_seconds += time.perf_counter() - t_begin
        self.launches += 1
        return bk.logits[:R], bk.tokens[:, :R]

    def run_portions(self, entries: List[StepEntry]) -> torch.Tensor:
        """A step with prompt portions from its bucket's graph; the head runs on the wanted rows afterwards.
        Returns float logits [wanted, V]."""
        t_begin = time.perf_counter()
        bk = self._portion_bucket(self._portion_size(sum(len(e.tokens) for e in entries)))
        d = self._fill_and_replay(bk, entries, 1)
        x, pending = bk.hidden
        logits = self.runner.model.head_logits(x, pending, bk.fields["logit_rows"][:d.logit_rows.size])
        self.enqueue_seconds += time.perf_counter() - t_begin
        self.launches += 1
        return logits


DecodeGraphs = StepGraphs   # the name this class had while it replayed decode steps only
