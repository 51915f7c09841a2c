"""The model's two ends: token embedding (a row gather into the float residual stream,
src/miniserve/model.py:229) and the output head (a matrix product with the head's own matrix or, when
tied, the embedding table, model.py:204-206, 237).  Logits are float."""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Embedding, Head, register_part


class TokenEmbedding(Embedding):
    def __init__(self, prefix: str, vocab_size: int, hidden_size: int):
        self.prefix, self.vocab_size, self.hidden_size = prefix, vocab_size, hidden_size

    def tensor_specs(self):
        return [TensorSpec(self.prefix + "weight", (self.vocab_size, self.hidden_size))]

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(self.tensor_specs()[0])

    def forward(self, ctx):
        out = self.rt.empty(ctx.num_tokens, self.hidden_size, dtype=torch.float32)
        return ops.embed(ctx.token_ids, self.weight, out)


class LMHead(Head):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, hidden_size: int, vocab_size: int, tied_to=None):
        self.prefix, self.hidden_size, self.vocab_size, self.tied_to = prefix, hidden_size, vocab_size, tied_to

    def tensor_specs(self):
        name = self.tied_to or self.prefix + "weight"
        return [TensorSpec(name, (self.vocab_size, self.hidden_size))]

    def ignorable(self):
        """A tied head ignores a copy of its own that the checkpoint may still carry."""
        return [self.prefix + "weight"] if self.tied_to else []

    def load(self, get, rt):
        self.rt = rt
        self.weight = linear.prepare_weight(get(self.tensor_specs()[0]))

    def forward(self, h):
        return linear.linear(h, self.weight, out_dtype=torch.float32)


register_part("embedding", "token_embedding", TokenEmbedding)
register_part("head", "lm_head", LMHead)
