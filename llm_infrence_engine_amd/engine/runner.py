"""The step function: run a batch of (request, its next tokens) from the cache and return the logits at
the wanted places.

One call = one forward of the model over exactly the tokens it is given: it allocates the pages they
need, writes their keys and values, attends over what earlier steps left, and commits the new lengths.
The reference's counterpart is ``Qwen2.forward(input_ids, cache=view, last_only)`` called once for a
prefill and once for the decode rows of a step (src/miniserve/paged_engine.py:126-127, 168-170).
"""
from __future__ import annotations

from typing import Hashable, List, Optional

import torch

from ..cache import CacheLayout, CacheManager, CachePools
from ..kernels import ops
from ..parts.model import Model, RunCache
from .batch import BatchBuilder, StepEntry


class ModelRunner:
    def __init__(self, model: Model, page_size: int, num_pages, max_requests: int, max_len: int,
                 hip_graphs: bool = False, graph_portion_tokens: Optional[int] = None):
        """``num_pages``: usable pages of every cache group's pool, or one number per group.  With ``hip_graphs``
        decode steps are replayed from captured graphs, and so are steps with prompt portions of up to
        ``graph_portion_tokens`` tokens (None: as far as the host would otherwise be what the step waits for)."""
        if model.rt is None:
            raise RuntimeError("the model has no weights yet; load it first")
        self.model, self.rt = model, model.rt
        self.layout = CacheLayout(model.run_needs())
        if len(self.layout.group_keys) > ops.MAX_CACHE_GROUPS:
            raise ValueError(f"the model's runs fall into {len(self.layout.group_keys)} cache groups; the kernels that "
                             f"keep block tables and slots serve at most {ops.MAX_CACHE_GROUPS}")
        self.manager = CacheManager(self.layout, page_size, num_pages, max_requests, max_len)
        self.pools = CachePools(self.layout, page_size, num_pages, max_requests, self.rt,
                                self.manager.max_pages_per_request)
        self.builder = BatchBuilder(self.manager, self.pools, model.spec.vocab_size, self.rt.device)
        self.graphs = None
        # a part that cannot be captured (it walks the requests on the host, as a mixer with state usually does)
        # keeps the whole model out of graphs
        if hip_graphs and model.graph_safe():
            from .graph import StepGraphs

            self.graphs = StepGraphs(self, portion_tokens=graph_portion_tokens)
        self.greedy_tokens: Optional[torch.Tensor] = None   # argmax of the last step's rows, if a graph computed it

    # ------------------------------------------------------------------ requests
    def add_request(self, req_id: Hashable) -> None:
        self.manager.add(req_id)

    def free_request(self, req_id: Hashable) -> None:
        self.manager.free(req_id)

    def caches(self, table_rows: torch.Tensor, slots) -> List[RunCache]:
        """What every run of the order is given for a step: its pages with its group's table and the step's slots,
        and its state slots."""
        out = []
        for i in range(len(self.model.spec.order)):
            g = self.layout.run_group[i]
            kv = self.pools.kv_view(i, table_rows, slots[g]) if g is not None else None
            state = self.pools.state_view(i) if i in self.layout.state_needs else None
            out.append(RunCache(kv, state))
        return out

    # ------------------------------------------------------------------ the step
    @torch.inference_mode()
    def step(self, entries: List[StepEntry]) -> torch.Tensor:
        """Float logits [wanted places, vocabulary], in the order of the entries and of their ``want``."""
        m = self.manager
        seen = set()
        for e in entries:
            if e.req_id in seen:
                raise ValueError(f"request {e.req_id!r} appears twice in one step")
            seen.add(e.req_id)
            if not m.has(e.req_id):
                m.add(e.req_id)
        for e in entries:
            m.grow(e.req_id, m.computed(e.req_id) + len(e.tokens))
        self.greedy_tokens = None
        kind = self.graphs.takes(entries) if self.graphs is not None else None
        if kind == "decode":
            logits, tokens = self.graphs.run(entries)
            wanted = [i for i, e in enumerate(entries) if len(e.want)]
            if len(wanted) == len(entries):
                self.greedy_tokens = tokens[0]
            else:        # replay only: a decoded token whose logits nobody asked for
                logits = logits[torch.tensor(wanted, dtype=torch.long, device=logits.device)] if wanted else logits[:0]
        elif kind == "portions":
            logits = self.graphs.run_portions(entries)
        else:
            built = self.builder.build(entries)
            logits = self.model.forward(built.ctx, self.caches(built.ctx.state_slots, built.slots))
        for e in entries:
            m.advance(e.req_id, m.computed(e.req_id) + len(e.tokens))
        return logits

    @torch.inference_mode()
    def decode_steps(self, entries: List[StepEntry], steps: int, sampling=None) -> List[List[int]]:
        """``steps`` decode steps in one launch of a captured graph: every request of ``entries`` (one token
        each, the one it is to be fed next) runs ``steps`` tokens ahead, each step fed the token the one before
        chose on the device: the argmax, or with ``sampling`` (one ``batch.Sampling`` per entry) a draw by each
        request's own rule, seed and count of draws.  Returns the chosen tokens, [steps][len(entries)]."""
        if self.graphs is None:
            raise RuntimeError("several decode steps per launch need hip_graphs")
        m = self.manager
        for e in entries:
            if len(e.tokens) != 1:
                raise ValueError("decode_steps takes one token per request")
            m.grow(e.req_id, m.computed(e.req_id) + steps)
        _, tokens = self.graphs.run(entries, steps, sampling)
        out = tokens.tolist()
        for e in entries:
            m.advance(e.req_id, m.computed(e.req_id) + steps)
        self.greedy_tokens = None
        return out


def load_runner(model_dir, dtype: str = "bfloat16", device: str = "cuda:0", page_size: int = 16,
                num_pages: Optional[int] = None, max_requests: int = 32, max_len: int = 1024,
                hip_graphs: bool = False, graph_portion_tokens: Optional[int] = None) -> ModelRunner:
    """Model folder -> a runner with an empty cache."""
    from ..loading import load_model

    model = load_model(model_dir, dtype, device)
    if num_pages is None:
        num_pages = max_requests * (-(-max_len // page_size))
    return ModelRunner(model, page_size, num_pages, max_requests, max_len, hip_graphs, graph_portion_tokens)
