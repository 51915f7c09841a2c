"""Matrix products of the model: out = a @ w.T (+ bias).  Picks the kernel by type and shape.

float32 always goes to the vector-ALU kernel (a true 32-bit product).  bfloat16 accumulates in float.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops


def prepare_weight(w: torch.Tensor) -> torch.Tensor:
    """The layout the kernels read: [out features, in features], rows contiguous."""
    return w.contiguous()


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    if out is None:
        out = torch.empty((a.shape[0], w.shape[0]), dtype=out_dtype or a.dtype, device=a.device)
    return ops.gemm_generic(a, w, out, bias=bias)
