"""Arrangements of a layer's parts.

``pre_norm_residual``: x = x + mixer(norm(x)); x = x + feed_forward(norm(x)) (src/miniserve/model.py:184-185).
The residual stream x is float; each sum is fused into the norm that follows it, so a block hands its
last addend on as ``pending``."""
from __future__ import annotations

from .base import Block, register_part


class PreNormResidual(Block):
    def forward(self, x, pending, ctx, kv, state):
        h = self.mixer_norm.forward(x, delta=pending)
        a = self.mixer.forward(h, ctx, kv, state)
        h = self.feed_forward_norm.forward(x, delta=a)
        return self.feed_forward.forward(h, ctx)


register_part("block", "pre_norm_residual", PreNormResidual)
