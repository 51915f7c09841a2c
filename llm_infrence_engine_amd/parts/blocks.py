"""Arrangements of a layer's parts.

``pre_norm_residual``: x = x + mixer(norm(x)); x = x + feed_forward(norm(x)) (src/miniserve/model.py:184-185).
The residual stream x is float.  A part either adds its result into x itself (its last matrix product does
it as an epilogue) or hands the addend on, and the sum is fused into the norm that follows; a block hands its
own last addend on as ``pending``."""
from __future__ import annotations

from .base import Block, register_part


class PreNormResidual(Block):
    takes = {"position": "position", "mixer_norm": "norm", "mixer": "mixer", "feed_forward_norm": "norm",
             "feed_forward": "feed_forward"}
    optional = ("position",)

    def forward(self, x, pending, ctx, kv, state):
        norm = self.mixer_norm.lazy if self.mixer.accepts_lazy_norm else self.mixer_norm.forward
        a = self.mixer.forward_residual(norm(x, delta=pending), ctx, kv, state, x)
        norm = self.feed_forward_norm.lazy if self.feed_forward.accepts_lazy_norm else self.feed_forward_norm.forward
        return self.feed_forward.forward_residual(norm(x, delta=a), ctx, x)


register_part("block", "pre_norm_residual", PreNormResidual)
