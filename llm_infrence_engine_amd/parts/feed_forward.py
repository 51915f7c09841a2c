"""Dense gated feed-forward: down(silu(gate(x)) * up(x)), no biases (src/miniserve/model.py:155-165).
Gate and up are one packed matrix product (rows interleaved so that the activation can be the product's
epilogue); the activation is float."""
from __future__ import annotations

from ..kernels import linear
from ..weights.spec import TensorSpec
from .base import FeedForward, register_part


class SwiGLU(FeedForward):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int):
        self.prefix, self.hidden_size, self.intermediate_size = prefix, hidden_size, intermediate_size

    def tensor_specs(self):
        p, H, I = self.prefix, self.hidden_size, self.intermediate_size
        return [TensorSpec(p + "gate_proj.weight", (I, H)), TensorSpec(p + "up_proj.weight", (I, H)),
                TensorSpec(p + "down_proj.weight", (H, I))]

    def load(self, get, rt):
        self.rt = rt
        g, u, d = (get(s) for s in self.tensor_specs())
        self.w_gate_up = linear.interleave_rows(g, u)
        self.w_down = linear.prepare_weight(d)

    def forward(self, h, ctx):
        return self.forward_residual(h, ctx, None)

    def forward_residual(self, h, ctx, x):
        return linear.linear_residual(linear.linear_swiglu(h, self.w_gate_up), self.w_down, None, x)


register_part("feed_forward", "swiglu", SwiGLU)
