from .base import (Block, Embedding, FeedForward, Head, KVNeed, KVView, Mixer, Norm, Part, PositionEncoding,
                   Runtime, StateNeed, StateView, StepContext, build_part, part_class, register_part)
from .model import Model, RunCache

__all__ = ["Block", "Embedding", "FeedForward", "Head", "KVNeed", "KVView", "Mixer", "Norm", "Part",
           "PositionEncoding", "Runtime", "StateNeed", "StateView", "StepContext", "build_part", "part_class",
           "register_part", "Model", "RunCache"]
