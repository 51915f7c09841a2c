"""RMS norm: y = weight * x * rsqrt(mean(x^2) + eps), computed in float on the float residual stream.

The reference computes the reduction in float, casts back and multiplies by the weight in the model's
type (src/miniserve/model.py:69-73); here the weight is applied in float too and the result is rounded once.
"""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import Norm, register_part


class RMSNorm(Norm):
    def __init__(self, prefix: str, size: int, eps: float):
        self.prefix, self.size, self.eps = prefix, size, eps

    def tensor_specs(self):
        return [TensorSpec(self.prefix + "weight", (self.size,), "norm")]

    def load(self, get, rt):
        self.rt = rt
        self.weight = get(self.tensor_specs()[0])

    def forward(self, x, delta=None, rows=None, write_back=True):
        n = x.shape[0] if rows is None else rows.numel()
        out = self.rt.empty(n, self.size)
        return ops.rms_norm(x, self.weight, self.eps, out, delta=delta, rows=rows, write_back=write_back)


    def lazy(self, x, delta=None, rows=None, write_back=True):
        """As ``forward``, for a consumer that can fold the norm into its first product: with few rows in
        bfloat16 the addend is summed into x now and the normalisation is left to that product."""
        n = x.shape[0] if rows is None else rows.numel()
        if self.rt.dtype != torch.bfloat16 or n > ops.SKINNY_MAX_ROWS or self.size % 8 or (delta is not None and not write_back):
            return self.forward(x, delta, rows, write_back)
        if delta is not None:
            ops.residual_add(x, delta)
        return linear.LazyNorm(x, self.weight, self.eps, self.rt.dtype, rows)


register_part("norm", "rms_norm", RMSNorm)
