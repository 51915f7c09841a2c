"""A model assembled from a ``ModelSpec``: embedding, layers in the order the spec gives, final norm, head.

The same layer may run more than once and a run may read an earlier run's cache; each run that keeps a
cache of its own is one entry of the cache manager's groups.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..config.spec import ModelSpec
from ..weights.reader import CheckpointReader, place
from ..weights.spec import TensorSpec
from . import attention, blocks, ends, feed_forward, norms, positions  # noqa: F401  (register the built-in parts)
from .base import KVView, Runtime, StateView, StepContext, build_part, part_class, weakest


@dataclass
class RunCache:
    """What one run of a layer was given by the cache manager for this step."""

    kv: Optional[KVView] = None
    state: Optional[StateView] = None


class Model:
    def __init__(self, spec: ModelSpec):
        self.spec = spec
        self.embedding = build_part("embedding", spec.embedding)
        self.layers = []
        for ls in spec.layers:
            self.layers.append(part_class("block", ls.block).build(ls.parts))
        self.final_norm = build_part("norm", spec.final_norm)
        self.head = build_part("head", spec.head)
        self.rt: Optional[Runtime] = None

    # ------------------------------------------------------------------ weights
    def _parts(self):
        return [self.embedding, *self.layers, self.final_norm, self.head]

    def tensor_specs(self) -> List[TensorSpec]:
        """Every tensor the model wants, each name once (a tied head names the embedding's)."""
        seen, out = set(), []
        for p in self._parts():
            for s in p.tensor_specs():
                if s.name not in seen:
                    seen.add(s.name)
                    out.append(s)
        return out

    def ignorable_tensors(self) -> List[str]:
        return list(getattr(self.head, "ignorable", lambda: [])())

    def load(self, reader: CheckpointReader, rt: Runtime) -> "Model":
        reader.check(self.tensor_specs(), self.ignorable_tensors())
        placed: Dict[str, torch.Tensor] = {}

        def get(spec: TensorSpec) -> torch.Tensor:
            if spec.name not in placed:
                placed[spec.name] = place(reader.get(spec.name), spec, rt.dtype, rt.device)
            return placed[spec.name]

        for p in self._parts():
            p.load(get, rt)
        self.rt = rt
        reader.close()
        return self

    # ------------------------------------------------------------------ cache needs, run by run
    def run_needs(self):
        """For every entry of the order: (CacheNeed or None, StateNeed(s) or None, cache_of)."""
        return [(self.layers[run.layer].cache_need(), self.layers[run.layer].state_need(), run.cache_of)
                for run in self.spec.order]

    def graph_safe(self):
        """Which steps of this model may be captured into graphs: True (all), "decode" (steps of single tokens)
        or False (none); the weakest answer of its parts (see ``Part.graph_safe``)."""
        return weakest([b.graph_safe() for b in self.layers] +
                       [p.graph_safe for p in (self.embedding, self.final_norm, self.head)])

    # ------------------------------------------------------------------ one step
    def forward(self, ctx: StepContext, caches: List[RunCache]) -> torch.Tensor:
        """Float logits [M, V] at ``ctx.logit_rows``.  Runs only the step's tokens, from the cache."""
        x, pending = self.forward_hidden(ctx, caches)
        return self.head_logits(x, pending, ctx.logit_rows)

    def forward_hidden(self, ctx: StepContext, caches: List[RunCache]):
        """Embedding and all runs of the order: the float residual stream [N, H] and the last run's addend that
        is still to be summed into it (or None)."""
        x = self.embedding.forward(ctx)
        pending = None
        for i, run in enumerate(self.spec.order):
            c = caches[i]
            pending = self.layers[run.layer].forward(x, pending, ctx, c.kv, c.state)
        return x, pending

    def head_logits(self, x: torch.Tensor, pending: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        """Final norm and head on the rows ``rows`` (int32) of what ``forward_hidden`` returned; x is left as it is."""
        if rows.numel() == 0:
            return torch.empty(0, self.spec.vocab_size, dtype=torch.float32, device=x.device)
        norm = self.final_norm.lazy if self.head.accepts_lazy_norm else self.final_norm.forward
        return self.head.forward(norm(x, delta=pending, rows=rows, write_back=False))
