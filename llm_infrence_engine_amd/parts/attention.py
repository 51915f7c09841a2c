"""Grouped-query attention over the paged cache.

q, k, v projections (one packed matrix product), position encoding fused with the cache store, causal
attention read in place from the pages, output projection.  Query head h uses key/value head
h // (num_heads // num_kv_heads) (src/miniserve/model.py:137-139).  Scores, softmax and the weighted
sum are float.  ``window`` limits a query to the last ``window`` keys (None: all).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..kernels import linear, ops
from ..weights.spec import TensorSpec
from .base import KVNeed, Mixer, register_part


class GQAttention(Mixer):
    accepts_lazy_norm = True

    def __init__(self, prefix: str, position, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 scale: float, qkv_bias: bool = True, out_bias: bool = False, window: Optional[int] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads cannot share {num_kv_heads} key/value heads")
        if head_dim % 16 or head_dim > 256:
            raise ValueError(f"head_dim {head_dim} is not supported: the attention kernels take multiples of 16 up to 256")
        if window is not None and window <= 0:
            raise ValueError("window must be positive")
        self.prefix, self.position = prefix, position
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.scale, self.qkv_bias, self.out_bias, self.window = float(scale), qkv_bias, out_bias, window

    # ---- weights
    def tensor_specs(self):
        p, H, d = self.prefix, self.hidden_size, self.head_dim
        specs = []
        for name, heads in (("q_proj", self.num_heads), ("k_proj", self.num_kv_heads), ("v_proj", self.num_kv_heads)):
            specs.append(TensorSpec(f"{p}{name}.weight", (heads * d, H)))
            if self.qkv_bias:
                specs.append(TensorSpec(f"{p}{name}.bias", (heads * d,), "bias"))
        specs.append(TensorSpec(f"{p}o_proj.weight", (H, self.num_heads * d)))
        if self.out_bias:
            specs.append(TensorSpec(f"{p}o_proj.bias", (H,), "bias"))
        if self.position is not None:
            specs += self.position.tensor_specs()
        return specs

    def load(self, get, rt):
        self.rt = rt
        by_name = {s.name: s for s in GQAttention.tensor_specs(self)}
        p = self.prefix
        w = [get(by_name[f"{p}{n}.weight"]) for n in ("q_proj", "k_proj", "v_proj")]
        self.w_qkv = linear.prepare_weight(torch.cat(w, dim=0))
        self.b_qkv = torch.cat([get(by_name[f"{p}{n}.bias"]) for n in ("q_proj", "k_proj", "v_proj")]).contiguous() \
            if self.qkv_bias else None
        self.w_o = linear.prepare_weight(get(by_name[f"{p}o_proj.weight"]))
        self.b_o = get(by_name[f"{p}o_proj.bias"]) if self.out_bias else None
        if self.position is not None:
            self.position.load(get, rt)

    # ---- cache
    def cache_need(self):
        # in bfloat16 the matrix-core attention reads value pages as an operand as they lie, transposed, which it
        # can for pages of a multiple of 16 tokens
        return KVNeed(self.num_kv_heads, self.head_dim, self.window, transpose_values_at=16,
                      transpose_values_in=torch.bfloat16)

    # ---- step
    def forward(self, h, ctx, kv, state):
        return self.forward_residual(h, ctx, kv, state, None)

    def forward_residual(self, h, ctx, kv, state, x):
        if kv is None:
            raise RuntimeError("attention needs a key/value cache view")
        nh, nkv, d = self.num_heads, self.num_kv_heads, self.head_dim
        q = None
        if self.position is not None:
            q = self.position.project_encode_store(h, self.w_qkv, self.b_qkv, nh, nkv, d, ctx, kv)
        if q is None:
            # [N, (nh + 2 nkv) d]: attention reads its q part.  A library product has no bias epilogue; a position
            # encoding that can add the bias on its way saves a pass over the projection.
            late_bias = (self.b_qkv is not None and getattr(self.position, "adds_bias", False)
                         and linear.goes_to_library(h, self.w_qkv))
            q = linear.linear(h, self.w_qkv, bias=None if late_bias else self.b_qkv)
            if late_bias:
                self.position.encode_and_store(q, nh, nkv, d, ctx, kv, bias=self.b_qkv)
            elif self.position is not None:
                self.position.encode_and_store(q, nh, nkv, d, ctx, kv)
            elif kv.store:
                ops.rope_store(q, nh, nkv, d, 0, None, None, kv.slot_mapping, kv.k_pages, kv.v_pages, kv.v_transposed)
        out = self.rt.empty(ctx.num_tokens, nh * d)
        ops.paged_attention(q, kv, ctx, out, nh, self.scale, self.window)
        return linear.linear_residual(out, self.w_o, self.b_o, x)


register_part("mixer", "gqa_attention", GQAttention)
