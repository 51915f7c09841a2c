"""Matrix products of the model: out = a @ w.T (+ bias).  Picks the kernel by type and shape.

float32          the vector-ALU kernel: a true 32-bit product, whatever the shape.
bfloat16, few rows (a decode step)   the weight-streaming matrix-core kernel, with the bias, the gated
                 activation or split-K partial sums as its epilogue.
bfloat16, many rows (prompt portions)  the library's matrix product (hipBLASLt through torch.mm), as the
                 reference uses a library for every product (F.linear, src/miniserve/model.py:123-165);
                 shapes it cannot take fall back to the vector-ALU kernel.  The gated gate/up product is
                 the tiled matrix-core kernel of our own where that is the faster one: its epilogue is
                 the activation, so the product itself is never written or read again.
All accumulate in float.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops

_mm_out_dtype_ok = None  # whether torch.mm can write float from bfloat16 inputs (found out at first use)

# Products that a few-rows kernel turned down (no block shape for the sizes) and that went to the vector-ALU
# kernel instead: correct, slower.  (shape, epilogue) -> times.  Zero for every shape the kernels are tuned for.
fallbacks = {}


def _fell_back(M: int, N: int, K: int, what: str) -> None:
    key = (M, N, K, what)
    fallbacks[key] = fallbacks.get(key, 0) + 1
    ops._say_once(("linear", N, K, what), f"no few-rows kernel for {what} of {M} x {K} by {N} x {K}; "
                                          f"the vector-ALU kernel runs it")


def fallback_count() -> int:
    return sum(fallbacks.values())


class LazyNorm:
    """Rows of the float residual stream that are still to be RMS-normalised.  The product that consumes them
    folds the norm in when it can (few rows, bfloat16 weights); otherwise ``materialize`` runs the norm kernel."""

    def __init__(self, x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype: torch.dtype,
                 rows: Optional[torch.Tensor] = None):
        self.x, self.weight, self.eps, self.out_dtype, self.rows = x, weight, eps, out_dtype, rows

    @property
    def num_rows(self) -> int:
        return self.x.shape[0] if self.rows is None else self.rows.numel()

    def materialize(self) -> torch.Tensor:
        out = torch.empty((self.num_rows, self.x.shape[1]), dtype=self.out_dtype, device=self.x.device)
        return ops.rms_norm(self.x, self.weight, self.eps, out, rows=self.rows)


def prepare_weight(w: torch.Tensor) -> torch.Tensor:
    """The layout the kernels read: [out features, in features], rows contiguous."""
    return w.contiguous()


def interleave_rows(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Rows a0, b0, a1, b1, ...: the packing of gate and up that the gated epilogue reads."""
    return torch.stack((a, b), dim=1).reshape(2 * a.shape[0], a.shape[1]).contiguous()


def _library_mm(a: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> Optional[torch.Tensor]:
    global _mm_out_dtype_ok
    if out_dtype == a.dtype:
        return torch.mm(a, w.t())
    if _mm_out_dtype_ok is None:
        try:
            torch.mm(a[:1], w[:1].t(), out_dtype=out_dtype)
            _mm_out_dtype_ok = True
        except (TypeError, RuntimeError):
            _mm_out_dtype_ok = False
    return torch.mm(a, w.t(), out_dtype=out_dtype) if _mm_out_dtype_ok else None


def goes_to_library(a, w: torch.Tensor) -> bool:
    """Whether ``linear(a, w)`` is a many-rows product, the library's or the tiled kernel's: both come without a
    bias epilogue."""
    return (isinstance(a, torch.Tensor) and a.dtype == torch.bfloat16 and not ops.skinny_ok(a, w)
            and a.shape[0] > ops.SKINNY_MAX_ROWS and a.is_contiguous())


def linear(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
           out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """[M, K] x [N, K] -> [M, N] in ``out_dtype`` (default: a's type).  ``a`` may be a ``LazyNorm``."""
    if isinstance(a, LazyNorm):
        if ops.skinny_norm_ok(a.x, w, a.num_rows) and ops.fold_norm_pays(a.num_rows, a.x.shape[1]):
            try:
                return ops.gemm_skinny_norm(a.x, a.weight, a.eps, w, bias, ops.EPI_STORE, out_dtype or a.out_dtype, a.rows)
            except ops.UnsupportedShape:
                _fell_back(a.num_rows, w.shape[0], w.shape[1], "norm + product")
        a = a.materialize()
    out_dtype = out_dtype or a.dtype
    if a.dtype == torch.bfloat16:
        if ops.skinny_ok(a, w):
            try:
                return ops.gemm_skinny(a, w, bias, ops.EPI_STORE, out_dtype=out_dtype)
            except ops.UnsupportedShape:
                _fell_back(a.shape[0], w.shape[0], w.shape[1], "product")
        if (a.shape[0] > ops.SKINNY_MAX_ROWS and out_dtype == torch.bfloat16 and bias is None
                and ops.gemm_tiled_plain_pays(a, w)):
            try:
                return ops.gemm_tiled(a, w)     # a short portion of a narrow model: the cheaper launch counts
            except ops.UnsupportedShape:
                _fell_back(a.shape[0], w.shape[0], w.shape[1], "tiled product")
        if a.shape[0] > ops.SKINNY_MAX_ROWS and a.is_contiguous():
            out = _library_mm(a, w, out_dtype)
            if out is not None:
                return ops.bias_add(out, bias) if bias is not None else out
    out = torch.empty((a.shape[0], w.shape[0]), dtype=out_dtype, device=a.device)
    return ops.gemm_generic(a, w, out, bias=bias)


def linear_residual(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                    residual: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """A product that is to be added to the float residual stream.  With few rows the kernel adds it into
    ``residual`` itself (each element by one lane, no atomics) and None is returned; otherwise the product
    [M, N] is returned for the next norm to add."""
    if residual is not None and a.dtype == torch.bfloat16 and ops.skinny_ok(a, w):
        try:
            ops.gemm_skinny(a, w, bias, ops.EPI_RESIDUAL, residual=residual)
            return None
        except ops.UnsupportedShape:
            _fell_back(a.shape[0], w.shape[0], w.shape[1], "product + residual")
            out = torch.empty((a.shape[0], w.shape[0]), dtype=a.dtype, device=a.device)
            return ops.gemm_generic(a, w, out, bias=bias)
    return linear(a, w, bias)


def linear_swiglu(a: torch.Tensor, w_gate_up: torch.Tensor) -> torch.Tensor:
    """silu(a @ gate.T) * (a @ up.T) for ``w_gate_up`` = interleave_rows(gate, up): [M, I].  ``a`` may be a
    ``LazyNorm``."""
    if isinstance(a, LazyNorm):
        if ops.skinny_norm_ok(a.x, w_gate_up, a.num_rows) and ops.fold_norm_pays(a.num_rows, a.x.shape[1]):
            try:
                return ops.gemm_skinny_norm(a.x, a.weight, a.eps, w_gate_up, None, ops.EPI_SWIGLU, rows=a.rows)
            except ops.UnsupportedShape:
                _fell_back(a.num_rows, w_gate_up.shape[0], w_gate_up.shape[1], "norm + gated product")
        a = a.materialize()
    if a.dtype == torch.bfloat16 and ops.skinny_ok(a, w_gate_up):
        try:
            return ops.gemm_skinny(a, w_gate_up, None, ops.EPI_SWIGLU)
        except ops.UnsupportedShape:
            _fell_back(a.shape[0], w_gate_up.shape[0], w_gate_up.shape[1], "gated product")
    if a.shape[0] > ops.SKINNY_MAX_ROWS and ops.gemm_tiled_pays(a, w_gate_up):
        try:
            return ops.gemm_tiled(a, w_gate_up, ops.EPI_SWIGLU)   # many rows: the activation is the product's epilogue
        except ops.UnsupportedShape:
            _fell_back(a.shape[0], w_gate_up.shape[0], w_gate_up.shape[1], "tiled gated product")
    gu = linear(a, w_gate_up)
    act = torch.empty((a.shape[0], w_gate_up.shape[0] // 2), dtype=a.dtype, device=a.device)
    return ops.silu_mul(gu, act)
