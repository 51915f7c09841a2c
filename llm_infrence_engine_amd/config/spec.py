"""What a model is made of, as data.

An architecture's typed configuration is turned into a ``ModelSpec``: a list of layers, each
naming its parts (mixer, feed-forward, norms, position encoding, arrangement) with their sizes
and constants, and the order in which the layers run.  Nothing below this file looks at an
architecture's configuration again; the parts are built from ``PartSpec`` alone.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: ``kind`` is its name in the part registry, ``prefix`` the beginning of its tensor
    names in the checkpoint, ``params`` its sizes and constants."""

    kind: str
    prefix: str = ""
    params: Mapping[str, Any] = field(default_factory=dict)


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which arrangement (``block``) puts which mixer and feed-forward behind which
    norms.  The position encoding belongs to the mixer (``position`` may be None)."""

    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    mixer_norm: PartSpec
    feed_forward_norm: PartSpec
    position: Optional[PartSpec] = None


@dataclass(frozen=True)
class Run:
    """One entry of the execution order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be
    named more than once: its weights are shared, each run has a cache of its own).  ``cache_of``
    names an earlier run whose cache this run reads instead of keeping one itself."""

    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    embedding: PartSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[Run, ...]
    final_norm: PartSpec
    head: PartSpec

    def __post_init__(self):
        for i, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{i}] names layer {run.layer}, but there are {len(self.layers)} layers")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ValueError(f"order[{i}] reads the cache of run {run.cache_of}, which does not come before it")
                if self.order[run.cache_of].cache_of is not None:
                    raise ValueError(f"order[{i}] reads the cache of run {run.cache_of}, which has none of its own")
