"""Rotary position encoding with half-split pairing.

inv_freq[j] = theta^(-2j/rotary_dim); the pair (j, j + rotary_dim/2) of every q and k head turns by
position * inv_freq[j] (src/miniserve/model.py:83-98).  Angles, sines and cosines are float in every
mode; the frequencies are derived in double on the host and rounded once.  The rotation is fused with
the store of k and v into the cache pages.
"""
from __future__ import annotations

import torch

from ..kernels import linear, ops
from .base import PositionEncoding, register_part


class RotaryHalf(PositionEncoding):
    adds_bias = True   # encode_and_store takes ``bias`` and adds it to q, k, v before rotating and storing

    def __init__(self, prefix: str, head_dim: int, rotary_dim: int, theta: float):
        if rotary_dim % 2 or not 0 < rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {rotary_dim} must be even and within head_dim {head_dim}")
        self.head_dim, self.rotary_dim, self.theta = head_dim, rotary_dim, float(theta)

    def load(self, get, rt):
        self.rt = rt
        j = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
        self.inv_freq = (1.0 / (self.theta ** (j / self.rotary_dim))).to(torch.float32).to(rt.device)

    def project_encode_store(self, h, w_qkv, bias, num_heads, num_kv_heads, head_dim, ctx, kv):
        if (kv is not None and kv.store
                and ops.gemm_tiled_qkv_pays(h, w_qkv, head_dim, self.rotary_dim, kv.k_pages)):
            # a portion of a prompt: rotation and cache store are the product's epilogue; the cosines and sines of
            # the step's positions are worked out by the first layer that comes here and shared by the others
            key = ("rotary_half", self.rotary_dim, self.theta)
            table = ctx.shared.get(key)
            if table is None:
                table = ctx.shared[key] = ops.rope_table(ctx.positions, self.inv_freq)
            return ops.gemm_tiled_qkv(h, w_qkv, bias, num_heads, num_kv_heads, head_dim, table, kv.slot_mapping,
                                      kv.k_pages, kv.v_pages, kv.v_transposed)
        if not (isinstance(h, linear.LazyNorm) and h.rows is None and kv is not None and kv.store
                and ops.qkv_rope_store_ok(h.x, w_qkv, head_dim, self.rotary_dim) and ops.qkv_rope_store_pays(h.x, w_qkv)):
            return None
        return ops.qkv_rope_store(h.x, h.weight, h.eps, w_qkv, bias, num_heads, num_kv_heads, head_dim, ctx.positions,
                                  self.inv_freq, kv.slot_mapping, kv.k_pages, kv.v_pages, kv.v_transposed)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv, bias=None):
        store = kv is not None and kv.store
        ops.rope_store(qkv, num_heads, num_kv_heads, head_dim, self.rotary_dim, ctx.positions, self.inv_freq,
                       kv.slot_mapping if store else None, kv.k_pages if store else None,
                       kv.v_pages if store else None, store and kv.v_transposed, bias)


class NoPosition(PositionEncoding):
    """No encoding: k and v are stored as they are."""

    def __init__(self, prefix: str = ""):
        pass

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, kv):
        if kv is not None and kv.store:
            ops.rope_store(qkv, num_heads, num_kv_heads, head_dim, 0, None, None, kv.slot_mapping, kv.k_pages,
                           kv.v_pages, kv.v_transposed)


register_part("position", "rotary_half", RotaryHalf)
register_part("position", "none", NoPosition)
