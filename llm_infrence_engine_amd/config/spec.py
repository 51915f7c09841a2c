"""What a model is made of, as data.

An architecture's typed configuration is turned into a ``ModelSpec``: a list of layers, each
naming its parts (mixer, feed-forward, norms, position encoding, arrangement) with their sizes
and constants, and the order in which the layers run.  Nothing below this file looks at an
architecture's configuration again; the parts are built from ``PartSpec`` alone.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from types import MappingProxyType
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True, eq=True)
class PartSpec:
    """One part: ``kind`` is its name in the part registry, ``prefix`` the beginning of its tensor
    names in the checkpoint, ``params`` its sizes and constants (kept read-only)."""

    kind: str
    prefix: str = ""
    params: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self):
        object.__setattr__(self, "params", MappingProxyType(dict(self.params)))

    def __hash__(self):
        return hash((self.kind, self.prefix, tuple(sorted((k, repr(v)) for k, v in self.params.items()))))


@dataclass(frozen=True, eq=True)
class LayerSpec:
    """One layer: an arrangement (``block``, a name in the block registry) and the parts it is given, by the
    names the arrangement takes (kept read-only).  ``pre_norm_residual`` takes ``mixer``, ``feed_forward``,
    ``mixer_norm``, ``feed_forward_norm`` and optionally ``position`` (the mixer's position encoding); another
    arrangement may take other parts (more norms, no feed-forward, two mixers).  ``layer.mixer`` is the part of
    that name; a name the layer was not given raises (``layer.parts.get(name)`` asks without raising)."""

    block: str
    parts: Mapping[str, PartSpec]

    def __post_init__(self):
        object.__setattr__(self, "parts", MappingProxyType(dict(self.parts)))

    def __hash__(self):
        return hash((self.block, tuple(sorted(self.parts.items(), key=lambda kv: kv[0]))))

    def __getattr__(self, name):
        if name.startswith("__") or name in ("block", "parts"):
            raise AttributeError(name)
        try:
            return self.parts[name]
        except KeyError:
            raise AttributeError(f"this {self.block} layer has no part named {name!r}; it has "
                                 f"{', '.join(sorted(self.parts))}") from None


def layer(block: str, **parts: Optional[PartSpec]) -> LayerSpec:
    """``LayerSpec`` from keyword parts; a part given as None is left out."""
    return LayerSpec(block, {k: v for k, v in parts.items() if v is not None})


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
