"""Plain, slow, whole-sequence Qwen2 decoder used only as the test oracle.

Written from the reference's formulas (citations are paths under the reference
checkout, ``src/miniserve/...``).  No cache, no batching tricks, one function per
part, and no import from the product package: it reads ``config.json`` and
``model.safetensors`` itself.  Everything runs in one floating type chosen by the
caller (float64 by default) so it can serve as the exact answer for both the
32-bit and the bfloat16 engine paths.
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import torch
from safetensors import safe_open


# --------------------------------------------------------------------------- files
def read_config(model_dir) -> dict:
    """The keys the reference reads (src/miniserve/model.py:42-58), with its defaults."""
    c = json.loads((Path(model_dir) / "config.json").read_text())
    rope = c.get("rope_theta")
    if rope is None:  # model.py:45-47
        rope = c.get("rope_parameters", {}).get("rope_theta", 10000.0)
    heads = c["num_attention_heads"]
    return {
        "vocab_size": c["vocab_size"],
        "hidden_size": c["hidden_size"],
        "intermediate_size": c["intermediate_size"],
        "num_layers": c["num_hidden_layers"],
        "num_heads": heads,
        "num_kv_heads": c["num_key_value_heads"],
        "rms_norm_eps": c["rms_norm_eps"],
        "rope_theta": float(rope),
        "tie_word_embeddings": c.get("tie_word_embeddings", False),
        # model.py:38-40 derives head_dim; a config may also state it
        "head_dim": c.get("head_dim") or c["hidden_size"] // heads,
    }


def read_weights(model_dir, dtype=torch.float64) -> dict:
    """All tensors of every ``*.safetensors`` file merged by name (src/miniserve/loader.py:41-43)."""
    out = {}
    for f in sorted(Path(model_dir).glob("*.safetensors")):
        with safe_open(str(f), framework="pt") as fh:
            for name in fh.keys():
                out[name] = fh.get_tensor(name).to(dtype)
    return out


# --------------------------------------------------------------------------- rounding
def rounded(x: torch.Tensor, act_dtype) -> torch.Tensor:
    """x as an engine that stores activations in ``act_dtype`` would hold it (None: exact).  Used only to
    measure how far a faithful reduced-precision computation strays from the exact one."""
    return x if act_dtype is None else x.to(act_dtype).to(x.dtype)


# --------------------------------------------------------------------------- parts
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2) + eps) * weight; eps inside the root (src/miniserve/model.py:69-73)."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(ms + eps))


def rope_inv_freq(head_dim: int, theta: float, dtype=torch.float64) -> torch.Tensor:
    """1 / theta^(2j/d), j = 0..d/2-1 (src/miniserve/model.py:83-85)."""
    return 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=dtype) / head_dim))


def rope_cos_sin(positions: torch.Tensor, head_dim: int, theta: float, dtype=torch.float64):
    """cos/sin tables [T, d]: angles pos * inv_freq, the half table repeated twice
    (src/miniserve/model.py:86-88)."""
    freqs = positions.to(dtype)[:, None] * rope_inv_freq(head_dim, theta, dtype)[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()


def rotate_half(x: torch.Tensor) -> torch.Tensor:
    """(-x2, x1) for x = (x1, x2) split in halves (src/miniserve/model.py:91-93)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x*cos + rotate_half(x)*sin; x is [heads, T, d], tables [T, d] (src/miniserve/model.py:96-98)."""
    return x * cos[None] + rotate_half(x) * sin[None]


def causal_attention(q, k, v, window=None) -> torch.Tensor:
    """softmax(q k^T / sqrt(d) + mask) v with grouped heads.

    q [nh, T, d]; k, v [nkv, S, d] with S == T here (whole sequence).  Query head h
    uses key/value head h // (nh // nkv) (repeat_interleave, src/miniserve/model.py:137-139);
    scale 1/sqrt(d) is the default of the library routine called at model.py:143; key j is
    visible to query i iff j <= i (model.py:143, cache.py:63-69).  ``window`` is not in the
    reference (it has no sliding window); when given, key j is also required to satisfy
    j > i - window, which is what the toy windowed layers of the tests use.
    """
    nh, T, d = q.shape
    nkv = k.shape[0]
    rep = nh // nkv
    k = k.repeat_interleave(rep, dim=0)
    v = v.repeat_interleave(rep, dim=0)
    scores = torch.einsum("htd,hsd->hts", q, k) / math.sqrt(d)
    i = torch.arange(T)[:, None]
    j = torch.arange(k.shape[1])[None, :]
    visible = j <= i
    if window is not None:
        visible = visible & (j > i - window)
    scores = scores.masked_fill(~visible[None], float("-inf"))
    return torch.einsum("hts,hsd->htd", torch.softmax(scores, dim=-1), v)


def attention_block(x, w, prefix, cfg, cos, sin, act_dtype=None) -> torch.Tensor:
    """Projections with q/k/v bias, rotation of q and k, attention, output projection without bias
    (src/miniserve/model.py:121-152)."""
    T = x.shape[0]
    nh, nkv, d = cfg["num_heads"], cfg["num_kv_heads"], cfg["head_dim"]
    q = x @ w[prefix + "q_proj.weight"].T + w[prefix + "q_proj.bias"]
    k = x @ w[prefix + "k_proj.weight"].T + w[prefix + "k_proj.bias"]
    v = x @ w[prefix + "v_proj.weight"].T + w[prefix + "v_proj.bias"]
    q = rounded(q, act_dtype).view(T, nh, d).transpose(0, 1)
    k = rounded(k, act_dtype).view(T, nkv, d).transpose(0, 1)
    v = rounded(v, act_dtype).view(T, nkv, d).transpose(0, 1)
    q = rounded(apply_rope(q, cos, sin), act_dtype)
    k = rounded(apply_rope(k, cos, sin), act_dtype)
    out = rounded(causal_attention(q, k, v), act_dtype)
    out = out.transpose(0, 1).reshape(T, nh * d)
    return rounded(out @ w[prefix + "o_proj.weight"].T, act_dtype)


def swiglu_mlp(x, w, prefix, act_dtype=None) -> torch.Tensor:
    """down(silu(gate(x)) * up(x)), no biases (src/miniserve/model.py:164-165)."""
    g = rounded(x @ w[prefix + "gate_proj.weight"].T, act_dtype)
    u = rounded(x @ w[prefix + "up_proj.weight"].T, act_dtype)
    return rounded(rounded(g * torch.sigmoid(g) * u, act_dtype) @ w[prefix + "down_proj.weight"].T, act_dtype)


def decoder_layer(x, w, i, cfg, cos, sin, act_dtype=None) -> torch.Tensor:
    """Two pre-norm residual branches (src/miniserve/model.py:184-185)."""
    p = f"model.layers.{i}."
    eps = cfg["rms_norm_eps"]
    h = rounded(rms_norm(x, w[p + "input_layernorm.weight"], eps), act_dtype)
    x = x + attention_block(h, w, p + "self_attn.", cfg, cos, sin, act_dtype)
    h = rounded(rms_norm(x, w[p + "post_attention_layernorm.weight"], eps), act_dtype)
    x = x + swiglu_mlp(h, w, p + "mlp.", act_dtype)
    return x


def forward(w: dict, cfg: dict, token_ids, position_offset: int = 0, act_dtype=None) -> torch.Tensor:
    """Logits [T, V] of one whole sequence (src/miniserve/model.py:222-237).

    ``position_offset`` shifts every position by a constant; the reference always starts at 0,
    the offset exists for the invariance test (only distances between positions matter).
    ``act_dtype`` (None: exact) rounds every activation that a reduced-precision engine stores between two
    kernels to that type, leaving the residual stream and the logits alone: a measure of the noise such an
    engine cannot avoid, never an expected value.
    """
    dtype = w["model.embed_tokens.weight"].dtype
    ids = torch.as_tensor(token_ids, dtype=torch.long)
    positions = torch.arange(len(ids)) + position_offset
    x = w["model.embed_tokens.weight"][ids]
    cos, sin = rope_cos_sin(positions, cfg["head_dim"], cfg["rope_theta"], dtype)
    for i in range(cfg["num_layers"]):
        x = decoder_layer(x, w, i, cfg, cos, sin, act_dtype)
    x = rounded(rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"]), act_dtype)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return x @ head.T


def greedy_generate(w: dict, cfg: dict, prompt, max_new_tokens: int, eos_ids=()) -> list:
    """Recompute-everything greedy decoding; the stop id is not emitted
    (src/miniserve/generate.py:69-82)."""
    ids = list(prompt)
    out = []
    for _ in range(max_new_tokens):
        tok = int(forward(w, cfg, ids)[-1].argmax())
        if tok in eos_ids:
            break
        out.append(tok)
        ids.append(tok)
    return out


# --------------------------------------------------------------------------- sampling
def logits_to_probs(logits: torch.Tensor, temperature=0.0, top_k=0, top_p=1.0) -> torch.Tensor:
    """The distribution tokens are drawn from (src/miniserve/sampler.py:12-41): temperature, then
    top-k (ties at the threshold kept), then top-p on the sorted tail (mass *before* a token
    >= top_p drops it), then softmax.  temperature <= 0 is one-hot on the first maximum."""
    logits = logits.to(torch.float64)
    if temperature <= 0.0:
        p = torch.zeros_like(logits)
        return p.scatter_(-1, logits.argmax(dim=-1, keepdim=True), 1.0)
    logits = logits / temperature
    if top_k > 0:
        kth = torch.topk(logits, min(top_k, logits.shape[-1])).values[..., -1, None]
        logits = logits.masked_fill(logits < kth, float("-inf"))
    if top_p < 1.0:
        srt, idx = torch.sort(logits, descending=True, dim=-1)
        probs = srt.softmax(dim=-1)
        before = probs.cumsum(dim=-1) - probs
        srt = srt.masked_fill(before >= top_p, float("-inf"))
        logits = torch.full_like(logits, float("-inf")).scatter(-1, idx, srt)
    return logits.softmax(dim=-1)
