from .base import (Block, CacheNeed, Embedding, FeedForward, Head, KVNeed, KVView, PageTensor, Mixer, Norm, Part, PositionEncoding,
                   Runtime, StateNeed, StateView, StepContext, build_part, part_class, register_part)
from .model import Model, RunCache

__all__ = ["Block", "CacheNeed", "PageTensor", "Embedding", "FeedForward", "Head", "KVNeed", "KVView", "Mixer", "Norm", "Part",
           "PositionEncoding", "Runtime", "StateNeed", "StateView", "StepContext", "build_part", "part_class",
           "register_part", "Model", "RunCache"]
