"""Interfaces of the parts a model is assembled from, and the registries that name them.

A part is built from the sizes and constants in its ``PartSpec`` alone and never learns which model
it is in.  Five kinds are chosen layer by layer:

``Norm``              forward(x, delta, rows, write_back) -> activations         (x: the float residual stream)
``PositionEncoding``  encode_and_store(qkv, nh, nkv, d, ctx, kv)                 (belongs to a mixer)
``Mixer``             forward(h, ctx, kv, state) -> [N, hidden]                  (attention here)
``FeedForward``       forward(h, ctx) -> [N, hidden]
                      (both also forward_residual(..., x): add into the residual stream x and return None,
                      or return the addend; the default returns forward's result)
``Block``             forward(x, pending, ctx, kv, state) -> pending             (the arrangement; it names the parts it takes)

plus ``Embedding`` and ``Head`` at the model's ends.  Every part lists the checkpoint tensors it wants
(``tensor_specs``) and takes them in ``load``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Tuple

import torch

from ..weights.spec import TensorSpec


# ------------------------------------------------------------------------------------------------ runtime data
@dataclass
class Runtime:
    """Where a model lives and the type of its matrices and activations."""

    device: torch.device
    dtype: torch.dtype

    def empty(self, *shape, dtype=None) -> torch.Tensor:
        return torch.empty(shape, dtype=dtype or self.dtype, device=self.device)


@dataclass(frozen=True)
class PageTensor:
    """One tensor of a cache page: ``heads`` x ``width`` values per token, kept as [heads, page_size, width].
    With ``transpose_at`` = n the pool keeps it as [heads, width, page_size] instead whenever the page size is
    a multiple of n (a mixer asks for that when its kernels read the tensor as a matrix operand as it lies),
    with ``transpose_in`` only when the cache holds that type.  What a part declares here does not depend on
    whether it has been loaded or in which type: the pool, which knows both, decides."""

    name: str
    heads: int
    width: int
    transpose_at: Optional[int] = None
    transpose_in: Optional[torch.dtype] = None


@dataclass(frozen=True)
class CacheNeed:
    """What a mixer keeps per token in pages: one or more tensors, for all tokens of a request (``window``
    None) or the last ``window`` of them.  Runs with equal needs share a group of the cache manager."""

    tensors: Tuple[PageTensor, ...]
    window: Optional[int] = None

    def __post_init__(self):
        names = [t.name for t in self.tensors]
        if not names or len(set(names)) != len(names):
            raise ValueError("a cache need names at least one page tensor, each name once")
        if self.window is not None and self.window <= 0:
            raise ValueError("window must be positive")

    def values_per_token(self) -> int:
        return sum(t.heads * t.width for t in self.tensors)


def KVNeed(num_kv_heads: int, head_dim: int, window: Optional[int] = None,
           transpose_values_at: Optional[int] = None, transpose_values_in: Optional[torch.dtype] = None) -> CacheNeed:
    """The usual need of attention: keys "k" and values "v", [num_kv_heads, head_dim] each."""
    return CacheNeed((PageTensor("k", num_kv_heads, head_dim),
                      PageTensor("v", num_kv_heads, head_dim, transpose_values_at, transpose_values_in)), window)


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request: one tensor of ``shape`` and ``dtype`` in a slot that the request holds
    from admission to its end.  The slot is zero when the request's first portion runs.  A mixer that keeps
    several such tensors returns a tuple of these."""

    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class KVView:
    """One run's pages of its cache group, with the group's block table and the step's slots.  The table lives
    on the device for as long as the cache does, one row per request the engine can hold (and a last row of
    null pages); request r of the step reads row ``table_rows[r]``."""

    pages: Dict[str, torch.Tensor]       # name -> [pages, heads, page_size, width], or [pages, heads, width, page_size]
    transposed: Dict[str, bool]          # name -> which of the two
    block_table: torch.Tensor            # int32 [rows, max pages]
    slot_mapping: torch.Tensor           # int32 [N]: page * page_size + offset of each token; < 0: not stored
    store: bool = True                   # False: the run reads another run's cache and writes nothing
    window: Optional[int] = None
    table_rows: Optional[torch.Tensor] = None   # int32 [R]; None: request r reads row r

    def pages_of(self, r: int) -> torch.Tensor:
        """The block-table row of the step's request ``r`` (for parts written in plain tensor code)."""
        return self.block_table[r if self.table_rows is None else self.table_rows[r].long()]

    # the usual pair of attention
    @property
    def k_pages(self) -> torch.Tensor:
        return self.pages["k"]

    @property
    def v_pages(self) -> torch.Tensor:
        return self.pages["v"]

    @property
    def v_transposed(self) -> bool:
        return self.transposed["v"]


@dataclass
class StateView:
    """One run's state slots: ``slots[state_slots[r]]`` belongs to request row r of the step.  ``slots`` is one
    tensor [num_slots, *shape], or a tuple of them when the mixer asked for several; the last slot is nobody's
    (rows that pad a batch point there)."""

    slots: object


@dataclass
class StepContext:
    """Everything a step's kernels need to know about its batch: N tokens of R requests, flattened.
    Device tensors are int32.  A request's tokens are consecutive; token n of request row r has absolute
    position ``positions[n]`` and sees the keys 0..positions[n] of that request."""

    num_tokens: int
    num_requests: int
    token_ids: torch.Tensor      # [N]
    positions: torch.Tensor      # [N]
    token_req: torch.Tensor      # [N] request row of each token
    q_start: torch.Tensor        # [R + 1] first token of each request's portion
    context_lens: torch.Tensor   # [R] keys each request holds once this step's tokens are stored
    state_slots: torch.Tensor    # [R] slot of each request's fixed-size state
    logit_rows: torch.Tensor     # [M] tokens whose logits are wanted
    max_q_len: int = 0           # an upper bound of the portions' lengths (the longest, outside a captured graph)
    max_context_len: int = 0     # and of the context lengths
    # [1], = q_start[R]: in a captured batch the tokens from there on belong to no request (None: there are none)
    n_live_tokens: Optional[torch.Tensor] = None
    # host copies for parts written in plain tensor code (tests' toy parts) and for kernel choice
    q_lens_host: List[int] = field(default_factory=list)
    start_pos_host: List[int] = field(default_factory=list)
    state_slots_host: List[int] = field(default_factory=list)
    # what a part derives from the step's tensors once for all layers that hold a part like it (key: the part's
    # choice); whoever changes ``positions`` in place empties it
    shared: dict = field(default_factory=dict)

    @property
    def decode_only(self) -> bool:
        return self.max_q_len == 1


# ------------------------------------------------------------------------------------------------ part interfaces
Getter = Callable[[TensorSpec], torch.Tensor]


def weakest(answers) -> object:
    """The least of several ``graph_safe`` answers: False < "decode" < True."""
    rank = {False: 0, "decode": 1, True: 2}
    worst = True
    for a in answers:
        a = a if a == "decode" else bool(a)
        if rank[a] < rank[worst]:
            worst = a
    return worst


class Part:
    # Whether a step that runs this part may be captured into a graph and replayed: the part reads the step's
    # batch from the device tensors of its StepContext only (never from the host copies, which a captured step
    # does not have), does not wait for the device and launches the same work whatever those tensors hold:
    # tokens dealt out over the requests in any way, requests without tokens and tokens of no request padding
    # the batch (``StepContext.n_live_tokens``).  True: every step; "decode": only steps in which every request
    # has one token (``ctx.decode_only``); False: none, and a model with such a part steps without graphs.
    graph_safe = True

    def tensor_specs(self) -> List[TensorSpec]:
        return []

    def load(self, get: Getter, rt: Runtime) -> None:
        """Take the tensors listed by ``tensor_specs`` (``get`` returns them placed on the device)."""
        self.rt = rt


class Norm(Part):
    def lazy(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None, rows: Optional[torch.Tensor] = None,
             write_back: bool = True):
        """What a block calls for a consumer that declares ``accepts_lazy_norm``: may return an object that
        the consumer's first product normalises on the fly (``kernels.linear.LazyNorm``).  Default: ``forward``."""
        return self.forward(x, delta, rows, write_back)

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None, write_back: bool = True) -> torch.Tensor:
        """Normalised activations of the float residual stream ``x`` [N, H].  With ``delta`` the sum
        x + delta is formed first (and kept in x unless ``write_back`` is False); with ``rows`` only
        those rows are produced."""
        raise NotImplementedError


class PositionEncoding(Part):
    def project_encode_store(self, h, w_qkv: torch.Tensor, bias: Optional[torch.Tensor], num_heads: int,
                             num_kv_heads: int, head_dim: int, ctx: StepContext, kv: Optional[KVView]):
        """Optional shortcut: projection, encoding and cache store in one kernel; returns q [N, nh d], or None
        when it cannot (then the mixer projects and calls ``encode_and_store``)."""
        return None

    def encode_and_store(self, qkv: torch.Tensor, num_heads: int, num_kv_heads: int, head_dim: int,
                         ctx: StepContext, kv: Optional[KVView]) -> None:
        """Encode positions into the q and k parts of ``qkv`` [N, (nh + 2 nkv) d] in place and, if ``kv``
        stores, put k and v into its pages.  A part with ``adds_bias = True`` also takes ``bias=`` (float
        [(nh + 2 nkv) d]) and adds it to q, k and v first."""
        raise NotImplementedError


class Mixer(Part):
    accepts_lazy_norm = False   # True: h may be a LazyNorm that the part hands to kernels.linear

    @property
    def graph_safe(self):
        """A mixer with per-request state is taken to walk its requests on the host unless its class says
        ``graph_safe = True`` or ``"decode"``."""
        return self.state_need() is None

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self):
        """None, a ``StateNeed``, or a tuple of them."""
        return None

    def forward(self, h: torch.Tensor, ctx: StepContext, kv: Optional[KVView],
                state: Optional[StateView]) -> torch.Tensor:
        raise NotImplementedError

    def forward_residual(self, h: torch.Tensor, ctx: StepContext, kv: Optional[KVView], state: Optional[StateView],
                         x: torch.Tensor) -> Optional[torch.Tensor]:
        """What the block calls.  A part whose last kernel can add into the float residual stream ``x`` does so
        and returns None; the default returns ``forward``'s result for the next norm to add."""
        return self.forward(h, ctx, kv, state)


class FeedForward(Part):
    accepts_lazy_norm = False

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        raise NotImplementedError

    def forward_residual(self, h: torch.Tensor, ctx: StepContext, x: torch.Tensor) -> Optional[torch.Tensor]:
        """As ``Mixer.forward_residual``."""
        return self.forward(h, ctx)


class Block(Part):
    """The arrangement of a layer's parts.  A block class names the parts it takes and their categories in
    ``takes`` (in the order their tensors are listed); ``LayerSpec.parts`` gives a ``PartSpec`` for each by
    name, those in ``optional`` may be missing.  A position encoding belongs to the mixer that is built after
    it (the mixer lists and loads its tensors).  ``pending`` is an addend of the residual stream that the
    previous layer left unsummed so that the next norm can fuse the sum; a block returns its own."""

    takes: Dict[str, str] = {}
    optional: Tuple[str, ...] = ()

    def __init__(self, **built):
        unknown = set(built) - set(self.takes)
        if unknown:
            raise TypeError(f"{type(self).__name__} takes {sorted(self.takes)}, not {sorted(unknown)}")
        self.built: Dict[str, Optional[Part]] = {}
        for name in self.takes:
            part = built.get(name)
            if part is None and name not in self.optional:
                raise TypeError(f"{type(self).__name__} needs a part named {name!r}")
            self.built[name] = part
            setattr(self, name, part)

    @classmethod
    def build(cls, specs) -> "Block":
        """Build every named part from its ``PartSpec`` and put them together."""
        unknown = set(specs) - set(cls.takes)
        if unknown:
            raise KeyError(f"the {cls.__name__} arrangement takes the parts {sorted(cls.takes)}; it has no {sorted(unknown)}")
        built: Dict[str, Optional[Part]] = {}
        position = None
        for name, category in cls.takes.items():
            spec = specs.get(name)
            if spec is None:
                if name not in cls.optional:
                    raise KeyError(f"the {cls.__name__} arrangement needs a part named {name!r}")
                built[name] = None
                continue
            extra = {"position": position} if category == "mixer" else {}
            built[name] = build_part(category, spec, **extra)
            if category == "position":
                position = built[name]
            elif category == "mixer":
                position = None
        return cls(**built)

    def parts(self) -> List[Part]:
        """The parts whose tensors the block lists and loads itself (position encodings go with their mixers)."""
        return [p for name, p in self.built.items() if p is not None and self.takes[name] != "position"]

    def mixers(self) -> List[Mixer]:
        return [p for p in self.built.values() if isinstance(p, Mixer)]

    def _caching_mixers(self) -> Dict[str, CacheNeed]:
        out = {}
        for name, p in self.built.items():
            if isinstance(p, Mixer):
                need = p.cache_need()
                if need is not None:
                    out[name] = need
        return out

    def cache_need(self) -> Optional[CacheNeed]:
        """What a run of this layer keeps per token.  One caching mixer: its need as it states it.  Several: one
        need that holds all their page tensors, each under ``<part name>.<tensor name>`` (a run has one cache
        group, so the mixers must keep their tokens for the same span); ``kv_of`` hands every mixer its own."""
        needs = self._caching_mixers()
        if len(needs) <= 1:
            return next(iter(needs.values()), None)
        windows = {n.window for n in needs.values()}
        if len(windows) > 1:
            raise ValueError(f"the caching mixers {sorted(needs)} of one layer keep their tokens for different spans "
                             f"({sorted(windows, key=str)}); the pages of a run are given back together")
        tensors = tuple(PageTensor(f"{name}.{t.name}", t.heads, t.width, t.transpose_at, t.transpose_in)
                        for name, need in needs.items() for t in need.tensors)
        return CacheNeed(tensors, windows.pop())

    def kv_of(self, name: str, kv: Optional[KVView]) -> Optional[KVView]:
        """The part of the run's cache view that belongs to the mixer ``name``, under the tensor names the mixer
        declared (the whole view when the layer has one caching mixer)."""
        if kv is None or len(self._caching_mixers()) <= 1:
            return kv
        prefix = name + "."
        return KVView({k[len(prefix):]: v for k, v in kv.pages.items() if k.startswith(prefix)},
                      {k[len(prefix):]: v for k, v in kv.transposed.items() if k.startswith(prefix)},
                      kv.block_table, kv.slot_mapping, kv.store, kv.window, kv.table_rows)

    def state_need(self):
        needs = []
        for m in self.mixers():
            n = m.state_need()
            if n is not None:
                needs.extend(n if isinstance(n, (tuple, list)) else [n])
        if not needs:
            return None
        return needs[0] if len(needs) == 1 else tuple(needs)

    def graph_safe(self):
        return weakest(p.graph_safe for p in self.built.values() if p is not None)

    def tensor_specs(self) -> List[TensorSpec]:
        return [s for p in self.parts() for s in p.tensor_specs()]

    def load(self, get: Getter, rt: Runtime) -> None:
        self.rt = rt
        for p in self.parts():
            p.load(get, rt)

    def forward(self, x: torch.Tensor, pending: Optional[torch.Tensor], ctx: StepContext,
                kv: Optional[KVView], state: Optional[StateView]) -> Optional[torch.Tensor]:
        raise NotImplementedError


class Embedding(Part):
    def forward(self, ctx: StepContext) -> torch.Tensor:
        """The float residual stream [N, H] of the step's tokens."""
        raise NotImplementedError


class Head(Part):
    accepts_lazy_norm = False

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        """Float logits [M, V] of normalised rows h [M, H]."""
        raise NotImplementedError


# ------------------------------------------------------------------------------------------------ registries
_REGISTRIES: Dict[str, Dict[str, type]] = {
    "norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(category: str, kind: str, cls: type) -> type:
    """Make ``cls`` buildable from ``PartSpec(kind=...)``.  Its constructor takes ``prefix`` and the spec's
    params as keywords (a mixer also ``position``, a built PositionEncoding or None)."""
    if category not in _REGISTRIES:
        raise KeyError(f"no part category {category!r}; there are {sorted(_REGISTRIES)}")
    _REGISTRIES[category][kind] = cls
    return cls


def part_class(category: str, kind: str) -> type:
    reg = _REGISTRIES[category]
    if kind not in reg:
        raise KeyError(f"no {category} part named {kind!r}; registered: {sorted(reg)}")
    return reg[kind]


def build_part(category: str, spec, **extra):
    return part_class(category, spec.kind)(prefix=spec.prefix, **dict(spec.params), **extra)
