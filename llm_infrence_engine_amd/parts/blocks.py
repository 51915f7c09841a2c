"""Arrangements of a layer's parts.

``pre_norm_residual``: x = x + mixer(norm(x)); x = x + feed_forward(norm(x)) (src/miniserve/model.py:184-185).
The residual stream x is float.  A part either adds its result into x itself (its last matrix product does
it as an epilogue) or hands the addend on, and the sum is fused into the norm that follows; a block hands its
own last addend on as ``pending``."""
from __future__ import annotations

from .base import Block, register_part


class PreNormResidual(Block):
    def forward(self, x, pending, ctx, kv, state):
        h = self.mixer_norm.forward(x, delta=pending)
        a = self.mixer.forward_residual(h, ctx, kv, state, x)
        h = self.feed_forward_norm.forward(x, delta=a)
        return self.feed_forward.forward_residual(h, ctx, x)


register_part("block", "pre_norm_residual", PreNormResidual)
